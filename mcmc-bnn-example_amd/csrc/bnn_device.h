// Structures shared by the host side of the library and its kernels.
#pragma once

#include <stdint.h>

namespace bnn {

// parameter layout, include/mcmc/mcmc_step_ffma.h:35-44
struct Layout {
  int d0, d1, oW1, ob1, ow2, ob2, P;
};
inline Layout make_layout(int d0, int d1) {
  Layout L;
  L.d0 = d0;
  L.d1 = d1;
  L.oW1 = 0;
  L.ob1 = d0 * d1;
  L.ow2 = L.ob1 + d1;
  L.ob2 = L.ow2 + d1;
  L.P = L.ob2 + 1;
  return L;
}

// float constants of the likelihood and the prior, derived on the host exactly as the reference
// derives them from its double constexprs (mcmc_step_ffma.h:289-300, 113-118)
struct ModelConsts {
  float scale;       // lik_scale
  float scale_recp;  // 1 / lik_scale
  float df;
  float df_recp;
  float lik_norm;  // Student-t or Gaussian normalisation
  float l_scale;   // -0.5 (df + 1)
  float g_scale;   // (df + 1) / scale
  float prior_recp;
  float prior_norm;
  float prior_neg_recp2;
};

enum KernelMode : int {
  MODE_STEPS = 0,       // L leapfrog steps from given (w, m, g): the step operator / evaluation
  MODE_TRANSITIONS = 1  // whole HMC transitions with RNG, accept, adaptation and sample store
};

// Number of floats of one workgroup's partial-result record: P gradient partials padded to a
// multiple of 4, then 4 words of which the first two hold a double (sum of per-row log-likelihood
// terms); rounded up to whole 128-byte lines so that a 32-parameter slice of a record is one line.
inline int partial_slot_floats(int P) { return (((P + 3) / 4) * 4 + 4 + 31) / 32 * 32; }

// 22 -> 40 -> 1 kernel, reduction by slices: the reducing workgroups publish the totals in up to this
// many identical copies (one per 32 workgroups of the group) and workgroup `rank` polls copy
// rank % copies, so that the polls of a group of 256 workgroups spread over eight times as many lines
// (polls of one line are served one after the other).
constexpr int TOTALS_COPIES = 8;

// status words at the start of the exchange scratch (64 are reserved)
constexpr int STATUS_WORDS = 64;

// 64-bit mixing function of the state hash (the finaliser of splitmix64)
#if defined(__HIPCC__)
__host__ __device__
#endif
inline unsigned long long mix64(unsigned long long z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// barrier words per chain group: the group's counter, eight block counters (one per 32 ranks, used by
// groups of more than 64 workgroups) and the counters of the second barrier of the two-phase
// reduction (arrivals, eight release lines), each on its own 128-byte line
constexpr int BARRIER_STRIDE_WORDS = 32 * 18;

struct KArgs {
  // ---- model / data ----
  int n;        // rows per window
  int n_tiles;  // ceil(n / 16)
  ModelConsts mc;
  const float* X;   // [window][n][d0]
  const float* y;   // [window][y_stride]
  long x_stride;    // floats between windows
  long y_stride;
  int x_vec_ok;     // X rows may be read with 8-byte loads
  int y_vec_ok;     // y may be read with 16-byte loads
  // ---- decomposition ----
  int G;            // workgroups per chain group
  int n_groups;     // chain groups in this launch
  int chain_base;   // global chain index of group 0
  int chain_wrap;   // > 0: chain indices wrap around at this count (group g runs chain (chain_base + g) mod it)
  int chains_per_window;
  int fixed_window; // >= 0: every group reads this window
  int xcd_map;      // 1: blockIdx is spread round-robin over 8 XCDs, keep a group inside one XCD
  int balance;      // 1: the two waves of a SIMD keep pace through wave priorities (prefetched loop)
  // ---- what to do ----
  int mode;
  int L;            // leapfrog steps per trajectory
  int n_trans;      // MODE_TRANSITIONS: transitions in this launch
  // ---- MODE_STEPS io (per group strides in floats; null inputs read as zero) ----
  const float* w_in;
  const float* m_in;
  const float* g_in;
  long in_stride;
  float* w_out;
  float* m_out;
  float* g_out;
  float* g_zero;      // zero-filled (the reference's grad_next)
  long out_stride;
  float* ell_out;     // per-row log-lik, [group][ell_stride]
  long ell_stride;
  float* prior_out;   // per-parameter log-prior, [group][out_stride]
  double* sums_out;   // [group][2]: sum of ell, sum of log-prior
  float eps_in;
  // ---- MODE_TRANSITIONS state, indexed by global chain ----
  float* st_w;        // [chain][PS]
  float* st_g;        // [chain][PS]
  long st_stride;
  float* st_eps;      // [chain]
  int* st_t;          // [chain] transitions done
  int* st_sel;        // [chain] which ell buffer holds the current state's rows
  int* st_nacc;       // [chain]
  float* ell0;        // [chain][ell_stride]
  float* ell1;
  float* samples;     // [chain][n_samples][P]
  int n_samples;
  int burn_in;
  int adapt_steps;
  float dec_adj;      // -decrement / (1 + decrement)
  float inc_adj;
  float log_target;   // log(target_rate)
  float* tr_log_acpt; // [chain][trace_len]
  int* tr_accept;
  float* tr_eps;
  int trace_len;
  uint32_t seed;
  uint32_t rng_id_base;  // RNG key word 1 of chain c is rng_id_base + c
  // ---- cross-workgroup exchange ----
  float* partials;     // [group][2][G][slot]; 22 -> 40 -> 1: slots of 8-byte packets {value, step number}
  float* totals;       // [group][slot]: reduced gradient, reduction by slices only
  int two_phase;       // 1: the first workgroups each reduce a slice of the parameters, then all read the totals
  unsigned* barrier;   // [group][BARRIER_STRIDE_WORDS], 64 -> 128 -> 1 only
  unsigned* status;    // [0] abort flag, [1] timed-out workgroup + 1; [4..9] belong to the hash check
  unsigned long long* rank_hash;  // [workgroup in group-major order]: hash of the state this workgroup
                                  // integrated; all workgroups of a chain group must agree
  unsigned spin_limit;
  float* wg_scratch;   // wide-layer kernel, MODE_TRANSITIONS: [workgroup][3][P_AL] accepted w, g and start momentum
  int debug_drop_rank; // >= 0: this rank of every group never publishes (exercises the timeout path)
  int debug_perturb_hash_rank;  // >= 0: this rank of every group flips a bit of its state hash
  unsigned* debug_xcc; // optional [workgroup] XCC id
  unsigned long long* debug_phase;  // optional [workgroup][10]: cycles per phase of a step, launch ticks
};

}  // namespace bnn
