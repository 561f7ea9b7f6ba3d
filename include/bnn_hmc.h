/*
 * bnn_hmc.h -- C ABI of the MI355X (gfx950) HMC sampler for the Bayesian 2-layer MLP.
 *
 * Every entry point replaces one piece of NVIDIA/mcmc-bnn-example; the reference interface it
 * stands in for is cited as file:line relative to the reference checkout.  Plain pointers and
 * sizes only.  All functions return BNNHMC_OK (0) or a BNNHMC_ERR_* code and never abort; the
 * message of the most recent failure on the calling thread is returned by bnnhmc_last_error().
 *
 * Parameter vector layout (include/mcmc/mcmc_step_ffma.h:35-44): theta = W1[k * d1 + c]
 * (k < d0 input, c < d1 hidden) | b1[c] | w2[c] | b2, P = d0*d1 + 2*d1 + 1 floats.
 *
 * Two levels:
 *   operator level -- caller-owned DEVICE buffers, same argument meaning as the reference's
 *                     device operators (mcmc_step, log_acpt_prec, the momentum lambda,
 *                     get_loss_values);
 *   sampler level  -- an opaque handle that owns all device memory and runs whole chains for many
 *                     windows on the GPU (the three phases of main_loop: init, run, dump).
 */
#ifndef BNN_HMC_H
#define BNN_HMC_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  BNNHMC_OK = 0,
  BNNHMC_ERR_INVALID = 1,   /* bad argument (null pointer, non-positive size, unsupported shape) */
  BNNHMC_ERR_HIP = 2,       /* a HIP runtime call failed                                          */
  BNNHMC_ERR_NO_DEVICE = 3, /* no gfx950 device visible                                           */
  BNNHMC_ERR_RESIDENCY = 4, /* the cooperating workgroups of one chain cannot all be resident     */
  BNNHMC_ERR_TIMEOUT = 5,   /* a bounded in-kernel wait expired; the launch was abandoned         */
  BNNHMC_ERR_STATE = 6,     /* call order violated (e.g. run before init_chains)                  */
  BNNHMC_ERR_DIVERGED = 7   /* the workgroups that share a chain did not all integrate the same   */
                            /* state (each reports a hash of it after every launch); the results  */
                            /* of the launch are not to be trusted                                */
};

enum { BNNHMC_LIK_STUDENT_T = 0, BNNHMC_LIK_GAUSSIAN = 1 };
enum { BNNHMC_LAYER_MFMA = 0, BNNHMC_LAYER_FFMA = 1 };

/* Model constants: include/mcmc/global_params.h:39-61 made runtime values. */
typedef struct bnnhmc_model {
  int d0;             /* input features, 22 (global_params.h:56)                        */
  int d1;             /* hidden units, 40 (global_params.h:56)                          */
  int n;              /* rows of the full batch, 58368 (global_params.h:61)             */
  int lik_kind;       /* BNNHMC_LIK_STUDENT_T (reference) or BNNHMC_LIK_GAUSSIAN        */
  double lik_scale;   /* Student-t scale 100 (global_params.h:39) or Gaussian sigma     */
  double lik_df;      /* Student-t degrees of freedom 2.2 (global_params.h:40)          */
  double prior_scale; /* Gaussian prior scale 200 (global_params.h:48)                  */
} bnnhmc_model;

/* Sampler constants: include/mcmc/global_params.h:27-36. */
typedef struct bnnhmc_hmc {
  int leapfrog_steps; /* 1000 */
  int burn_in;        /* 100  */
  int n_samples;      /* 800  */
  int adapt_steps;    /* = burn_in */
  float eps0;         /* 0.01 */
  float target_rate;  /* 0.2  */
  float decrement;    /* 0.1  */
  float increment;    /* 0.01 */
  uint32_t seed;      /* RNG key word 0; key word 1 is the global chain index */
  uint32_t chain_id_base; /* global index of this sampler's chain 0 (default 0): a sampler that  */
                      /* holds a slice of a larger job draws the streams the whole job would  */
} bnnhmc_hmc;

/* How the work is laid over the GPU.  Zero in a field selects the default. */
typedef struct bnnhmc_launch {
  int layer;          /* BNNHMC_LAYER_MFMA (v_mfma_f32_16x16x4_f32, _4x4x1_16b_f32) or BNNHMC_LAYER_FFMA */
  int cus_per_chain;  /* workgroups that share one chain's rows; 0 = automatic.  Sampler,         */
                      /* 22 -> 40 -> 1: a batch is the largest power-of-two number of chains that */
                      /* fits, spread over the whole device (one chain: 256 workgroups; 128 or     */
                      /* more chains on 256 CUs: 2 each) -- or, where that is measured to be       */
                      /* faster, the largest whose windows' rows stay within 358 MB, most of       */
                      /* which the memory-side cache serves (64 windows of 58368 x 22: 4 each; see */
                      /* bnnhmc_get_batching); more chains than fit take turns on such             */
                      /* batches, transitions_per_launch transitions at a time, and what does not  */
                      /* fill a batch runs in smaller, wider ones.  64 -> 128 -> 1: 4, a smaller    */
                      /* last batch widened.  Step operator: 256.  Results are bit-reproducible for */
                      /* a fixed count; with 0 and more chains than fit at once, which launches run */
                      /* wider depends on how a job is cut into bnnhmc_run calls and on that time   */
                      /* measurement, so a run that must be repeatable or resumable bit for bit     */
                      /* sets an explicit count                                                     */
  int wgs_per_cu;     /* co-resident workgroups per CU, 1 or 2 (default 1)                       */
  int threads;        /* threads per workgroup; default 512 for MFMA (every tile loop), 256 for  */
                      /* FFMA and with wgs_per_cu = 2.  The plain MFMA loop is also built for    */
                      /* 256, 768 and 1024 threads (the last two leave too few registers and    */
                      /* spill: correct, slower)                                                 */
  int pipeline;       /* MFMA tile loop: 0 = default: loop 4 at 512 threads, loop 3 otherwise;   */
                      /* 4 = loads issued two tiles ahead with explicit waits, hidden units      */
                      /* 32 .. 39 on v_mfma_f32_4x4x1_16b_f32 blocks (512 threads only: asking   */
                      /* for it with another size is an error), 2 = the same loop with three     */
                      /* 16-wide hidden tiles (the last one half empty; 512 threads only),       */
                      /* 1 = software-pipelined GEMM/pointwise stages (512 or 256 threads),      */
                      /* 3 = plain loop (256, 512, 768 or 1024 threads)                          */
  int transitions_per_launch; /* bound on one kernel's run time (default 5; 1 for 64 -> 128 -> 1);       */
                              /* times leapfrog_steps it must stay below 2^32 - 1                        */
  unsigned spin_limit; /* polls before an in-kernel wait gives up (default 1 << 22)              */
} bnnhmc_launch;

void bnnhmc_default_model(bnnhmc_model* m);   /* global_params.h:39-61 */
void bnnhmc_default_hmc(bnnhmc_hmc* h);       /* global_params.h:27-36 */
void bnnhmc_default_launch(bnnhmc_launch* l);
int bnnhmc_num_params(int d0, int d1);        /* global_params.h:58 */
const char* bnnhmc_last_error(void);
/* number of visible devices and, for device 0, its compute units and gcn arch name */
int bnnhmc_device_info(int* n_devices, int* compute_units, char* arch, size_t arch_len);

/* ------------------------------------------------------------------------------------------------
 * Operator level.  Pointers are DEVICE pointers owned by the caller; `stream` is a hipStream_t
 * (NULL = default stream).  Calls are asynchronous on `stream` unless stated.
 * ---------------------------------------------------------------------------------------------- */

/* Device scratch the step operator needs (per-workgroup gradient records, status words); the
 * counterpart of the reference's grid_sync_workspace (include/mcmc/main.h:171,
 * include/mcmc/mcmc_step_tc.h:597-612).  The workspace must be 16-byte aligned (any hipMalloc
 * result is). */
size_t bnnhmc_step_workspace_bytes(const bnnhmc_model* model, const bnnhmc_launch* launch);

/* How the step operator lays one chain over the GPU: workgroups, threads per workgroup, the most rows a
 * wavefront takes, LDS bytes of a workgroup and the most a workgroup may use.  Stands in for the
 * compile-time constants N_BLKS, N_THREADS, N_WARP_SAMPLES and for full_smem_size<T>() /
 * leapfrog_max_smem_size<T>() that the reference's driver prints (include/mcmc/main.h:120-125;
 * include/mcmc/mcmc_step_ffma.h:46-70).  Any output may be NULL.  Needs a device. */
int bnnhmc_step_launch_info(const bnnhmc_model* model, const bnnhmc_launch* launch, int* workgroups,
                            int* threads, int* rows_per_wave, size_t* lds_bytes, size_t* lds_max_bytes);

/* L fused leapfrog steps.  Replaces mcmc::mcmc_step<T, LP_STEPS>
 * (include/mcmc/mcmc_step_ffma.h:395-427, include/mcmc/mcmc_step_tc.h:679-696).
 * In : weights_prev, mom_prev, grad_prev (full gradient of the log-posterior at weights_prev), eps.
 * Out: weights_next; mom_next (lacking the final half kick, which the accept formula applies);
 *      grad_cur (full gradient at weights_next); grad_next zeroed; loss_values[n + P] = per-row
 *      log-likelihood then per-parameter log-prior at weights_next.  Unlike the reference's FFMA
 *      variant no caller pointers are rotated: results always land in the buffers named here. */
int bnnhmc_mcmc_step(const bnnhmc_model* model, const bnnhmc_launch* launch, const float* x,
                     const float* y, const float* weights_prev, float* weights_next,
                     const float* mom_prev, float* mom_next, const float* grad_prev,
                     float* grad_cur, float* grad_next, float* loss_values, void* workspace,
                     size_t workspace_bytes, float eps, int lp_steps, void* stream);

/* bnnhmc_mcmc_step for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): the same operator with the same arguments
 * but no workspace -- the exchange scratch is a static device array inside the library (4.5 MiB on
 * every GPU the library runs on, held until the process ends), and the call allocates nothing.  It
 * has no counterpart in the reference.  Configurations whose scratch would not fit (see
 * bnnhmc_step_workspace_bytes) are refused with BNNHMC_ERR_INVALID.  All calls on one GPU share the
 * array: calls that overlap on one GPU (two streams, two threads) race; calls issued one after the
 * other on one stream do not.  Check the outcome with bnnhmc_step_check(model, launch, NULL, stream).
 * The first call for a (device, model, launch) configuration looks up device properties, the kernel's
 * occupancy and the array's address, none of which may be asked for while a stream is capturing: make
 * one call per configuration outside capture first; every later call only launches kernels. */
int bnnhmc_mcmc_step_static(const bnnhmc_model* model, const bnnhmc_launch* launch, const float* x,
                            const float* y, const float* weights_prev, float* weights_next,
                            const float* mom_prev, float* mom_next, const float* grad_prev,
                            float* grad_cur, float* grad_next, float* loss_values, float eps,
                            int lp_steps, void* stream);

/* Synchronises `stream` and reports whether every bnnhmc_mcmc_step on this workspace since the last
 * check ran to completion: BNNHMC_ERR_TIMEOUT if a bounded in-kernel wait expired (the outputs of that
 * step were then not written, and steps queued behind it may have been abandoned too),
 * BNNHMC_ERR_DIVERGED if the workgroups did not all hold the same state at the end of a step.  The
 * record of a failure stays in the workspace until this call has reported it (and then clears it), so
 * one check after a whole sequence of steps is enough.
 * `launch` is not needed (the record sits at the start of the workspace) and may be NULL; workspace
 * NULL means the library's own scratch (bnnhmc_mcmc_step_static) on the current GPU.  Stands in
 * for the CUDA_CHECK after the launch (include/mcmc/mcmc_step_ffma.h:412). */
int bnnhmc_step_check(const bnnhmc_model* model, const bnnhmc_launch* launch, void* workspace,
                      void* stream);

/* Momentum resampling: prev_lp_mom[i] = mom_next[i] ~ N(0,1), i < n, for transition `transition`
 * of chain `chain_id`.  Replaces the eltWiseApply lambda at include/mcmc/main.h:207-216 (counter
 * based generator instead of thrust::minstd_rand + discard). */
int bnnhmc_sample_momentum(uint32_t seed, uint32_t chain_id, uint32_t transition, int n,
                           float* prev_lp_mom, float* mom_next, void* stream);

/* Log accept ratio: sum_i (new_loss[i] - prev_loss[i]), i < n_loss, plus
 * sum_i 0.5 (prev_mom[i]^2 - (new_mom[i] + 0.5 eps grad_cur[i])^2), i < n_mom.  Replaces
 * log_acpt_prec (include/mcmc/kernel_helpers.h:153-188).  Writes the value to log_acpt_out (device,
 * may be NULL) and, if host_out is not NULL, copies it to the host and synchronises the stream as
 * the reference does. */
int bnnhmc_log_acpt(int n_loss, int n_mom, const float* prev_loss, const float* new_loss,
                    const float* prev_mom, const float* new_mom, const float* grad_cur, float eps,
                    float* log_acpt_out, float* host_out, void* stream);

/* Sums of the data log-likelihood (first n entries) and of the log-prior (next n_params entries) of
 * a loss_values vector.  Replaces get_loss_values (include/mcmc/kernel_helpers.h:190-216);
 * synchronises the stream.  Allocates nothing; at most 64 calls may be in flight at once on a GPU. */
int bnnhmc_get_loss_values(const float* loss_values, int n, int n_params, float* loss1_host,
                           float* loss2_host, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Sampler level: the phases of mcmc::main_loop (include/mcmc/main.h:117-308) for many windows.
 * Host pointers unless stated.  A sampler is bound to device 0 and one stream; calls on one sampler
 * are not thread-safe, distinct samplers are independent.
 * ---------------------------------------------------------------------------------------------- */
typedef struct bnnhmc_sampler bnnhmc_sampler;

/* init, part 1: allocate state for n_windows * chains_per_window chains (main.h:156-183). */
int bnnhmc_create(const bnnhmc_model* model, const bnnhmc_hmc* hmc, const bnnhmc_launch* launch,
                  int n_windows, int chains_per_window, bnnhmc_sampler** out);
int bnnhmc_destroy(bnnhmc_sampler* s);

/* init, part 2: upload one window's features x[n][d0] and targets y[n] (read_data + copies,
 * include/mcmc/io.h:43-86; the caller applies any feature scaling, main.h:162-164). */
int bnnhmc_set_window_data(bnnhmc_sampler* s, int window, const float* x, const float* y);
/* ... or fill it with the benchmark's synthetic recipe: x ~ N(0,1), teacher weights
 * ~ N(0, teacher_scale^2), y = MLP_teacher(x) + N(0, noise_sigma^2), all from key (seed, window).
 * teacher_out (P floats) may be NULL. */
int bnnhmc_generate_window(bnnhmc_sampler* s, int window, float teacher_scale, float noise_sigma,
                           float* teacher_out);
/* the same recipe on the host only (no GPU needed): x_out[n][d0], y_out[n], teacher_out[P] or NULL */
int bnnhmc_generate_window_host(uint32_t seed, uint32_t window, int n, int d0, int d1,
                                float teacher_scale, float noise_sigma, float* x_out, float* y_out,
                                float* teacher_out);
/* host evaluation of the generator the device uses: 32-bit word `index` of stream
 * (stream, t) under key (seed, id); stream ids 0 features, 1 teacher, 2 noise, 3 momentum,
 * 4 accept uniform.  The momentum of parameter p at transition t of chain c is
 * bnnhmc_rng_normal(seed, c, 3, t, p); the accept test compares bnnhmc_rng_log_uniform(seed, c, t)
 * with the log accept ratio (main.h:235-242). */
uint32_t bnnhmc_rng_word(uint32_t seed, uint32_t id, uint32_t stream, uint32_t t, uint64_t index);
float bnnhmc_rng_normal(uint32_t seed, uint32_t id, uint32_t stream, uint32_t t, uint64_t index);
float bnnhmc_rng_log_uniform(uint32_t seed, uint32_t chain_id, uint32_t t);
/* Parse the reference's dataset text file (read_data, include/mcmc/io.h:43-86): one header line of
 * total_cols tokens, then per row total_cols tokens of which the first skip_cols are ignored, the next
 * one is the label and the next d0 are the features.  x_out[n][d0], y_out[n].  Host only.  The
 * reference's constants are total_cols = 149, skip_cols = 2 (global_params.h:63-65); its x0.001
 * feature scaling (main.h:162-164) is left to the caller. */
int bnnhmc_read_reference_data(const char* path, int n, int d0, int total_cols, int skip_cols,
                               float* x_out, float* y_out);
/* read back a window's data (x_out[n][d0], y_out[n]; either may be NULL) */
int bnnhmc_get_window_data(bnnhmc_sampler* s, int window, float* x_out, float* y_out);

/* init, part 3: set every chain to w0 (P floats, NULL = zeros as main.h:52,182), eps = eps0, and
 * evaluate the log-posterior and its gradient there (the bootstrap step, main.h:191-202). */
int bnnhmc_init_chains(bnnhmc_sampler* s, const float* w0);

/* run: n_transitions HMC transitions of every chain -- momentum resampling, the fused trajectory,
 * the log accept ratio, the Metropolis decision, step-size adaptation and the sample store
 * (main.h:204-287) -- entirely on the device.  Synchronous at return. */
int bnnhmc_run(bnnhmc_sampler* s, int n_transitions);

/* dump: kept samples of one chain, samples_out[n_stored][P] in transition order (main.h:277-283,
 * 295); n_stored may be NULL. */
int bnnhmc_get_samples(bnnhmc_sampler* s, int chain, float* samples_out, int* n_stored);
/* current state of one chain; any output may be NULL */
int bnnhmc_get_chain_state(bnnhmc_sampler* s, int chain, float* w, float* grad, float* eps,
                           int* transitions_done, int* n_accepted);
/* Overwrite the state of one chain (checkpoint resume): position w (P floats), step size, number of
 * transitions already done (selects the RNG counters and the sample slots) and of accepted ones.  The
 * log-posterior rows and the gradient at w are re-evaluated, which reproduces the bits a run that
 * never stopped would hold, so the continuation is exact.  No reference counterpart (the reference
 * keeps no checkpoint). */
int bnnhmc_set_chain_state(bnnhmc_sampler* s, int chain, const float* w, float eps,
                           int transitions_done, int n_accepted);
/* per-transition traces of one chain, each of length transitions_done; any may be NULL */
int bnnhmc_get_traces(bnnhmc_sampler* s, int chain, float* log_acpt, int* accepted, float* eps);

/* Log-posterior pieces at w (P floats) on one window's data: ell[n] per-row log-likelihood,
 * prior[P] per-parameter log-prior, grad[P] full gradient; any output may be NULL.  This is
 * mcmc_step<T,1> with eps = 0 as used by output_final_loss (main.h:92-99). */
int bnnhmc_eval(bnnhmc_sampler* s, int window, const float* w, float* ell, float* prior,
                float* grad);
/* Mean over one chain's kept samples of the data log-likelihood, the log-prior and their sum
 * (output_final_loss, main.h:78-115). */
int bnnhmc_final_loss(bnnhmc_sampler* s, int chain, double* loss1, double* loss2, double* full);

/* How bnnhmc_run lays the sampler's chains over the device at present: chains in a full launch and
 * workgroups per chain in it.  With the automatic group size (cus_per_chain = 0) of the 22 -> 40 -> 1 kernel
 * a launch takes the largest power-of-two number of chains that fits the device at one workgroup per chain;
 * where the rows of so many windows exceed 358 MB (1.4 times the memory-side cache, which serves most of a
 * batch of that size because a wave walks its tiles back and forth) there is a second shape, the largest
 * such number whose windows' rows stay within 358 MB (200 windows of 58368 x 22: 64 at a time on 4
 * workgroups each, against 128 on 2).  Which is faster depends on the card and on the data (the card is
 * power-limited: HBM traffic costs shader clock when the arithmetic is dense).  A sampler starts with the
 * shape within the budget; a bnnhmc_run call that is long enough (a launch of each shape fits in it) first
 * runs one launch of each, timed, and goes on with the faster, and so do later calls, which time the two
 * again after every 2000 launches' worth of chains.  trial_rates (may be NULL) receives the gradient
 * evaluations per second of the last such pair, the shape within the budget first; zeros if none was run.
 * No counterpart in the reference (one chain per process). */
int bnnhmc_get_batching(bnnhmc_sampler* s, int* chains_per_launch, int* workgroups_per_chain,
                        double* trial_rates);

/* Timing of the work done by bnnhmc_run so far: milliseconds between HIP events recorded on the
 * sampler's stream around the trajectory kernels, number of those launches, gradient evaluations
 * they performed (chains * transitions * leapfrog_steps), and the workgroups of the last launch. */
int bnnhmc_get_timing(bnnhmc_sampler* s, double* kernel_ms, long* launches, long* grad_evals,
                      int* workgroups);

/* ------------------------------------------------------------------------------------------------
 * Convergence diagnostics over the chains of one window (host arithmetic in double precision).
 * No counterpart in the reference, which runs one chain per window and prints only the final
 * losses (main.h:295-307); the scaled benchmark shape runs four chains per window, which is what
 * these need.  Estimators of Gelman et al., Bayesian Data Analysis 3rd ed., section 11.4-11.5, as
 * refined by Vehtari et al. 2021 (without rank normalisation):
 *   every chain is split in halves (m = 2 * n_chains sequences of n = n_samples / 2 draws),
 *   W = mean within-sequence variance, B / n = variance of the sequence means,
 *   var+ = (n - 1) / n * W + B / n,   rhat = sqrt(var+ / W),
 *   rho_t = 1 - (W - mean_j acov_j(t)) / var+,   ess = m n / (-1 + 2 sum_t P_t),
 * where P_t = rho_2t + rho_2t+1 runs over Geyer's initial positive sequence, made monotone.
 * A parameter that does not vary (W = 0) reports rhat = 1 and ess = m n.
 * ---------------------------------------------------------------------------------------------- */

/* samples[chain * chain_stride + draw * n_params + p] on the host; rhat and ess receive n_params
 * doubles each (either may be NULL).  Needs n_chains >= 1 and n_samples >= 8.  No GPU involved. */
int bnnhmc_split_rhat_ess(const float* samples, int n_chains, int n_samples, int n_params,
                          size_t chain_stride, double* rhat, double* ess);
/* The same over the kept samples of the chains of `window` of a sampler. */
int bnnhmc_window_diagnostics(bnnhmc_sampler* s, int window, double* rhat, double* ess);

#ifdef __cplusplus
}
#endif
#endif
