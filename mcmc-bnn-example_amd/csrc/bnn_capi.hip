// Host side of the C ABI declared in include/bnn_hmc.h.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <thread>
#include <vector>

#include "bnn_device.h"
#include "bnn_hmc.h"
#include "bnn_kernels.h"
#include "bnn_rng.h"

namespace {

using namespace bnn;

thread_local std::string g_last_error;

int fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

#define HIP_TRY(expr)                                                                      \
  do {                                                                                     \
    hipError_t e_ = (expr);                                                                \
    if (e_ != hipSuccess)                                                                  \
      return fail(BNNHMC_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_),   \
                  __FILE__, __LINE__);                                                     \
  } while (0)

// float constants from the double model constants, as the reference's lit<T>(double expr) does
// (mcmc_step_ffma.h:289-300, 113-118; global_params.h:41-52)
ModelConsts make_consts(const bnnhmc_model& m) {
  const double pi = 3.14159265358979323846;
  ModelConsts c;
  c.scale = (float)m.lik_scale;
  c.scale_recp = (float)(1.0 / m.lik_scale);
  c.df = (float)m.lik_df;
  c.df_recp = m.lik_kind == BNNHMC_LIK_STUDENT_T ? (float)(1.0 / m.lik_df) : 0.0f;
  if (m.lik_kind == BNNHMC_LIK_STUDENT_T) {
    c.lik_norm = (float)(std::log(std::fabs(m.lik_scale)) + 0.5 * std::log(m.lik_df) +
                         0.5 * std::log(pi) + std::lgamma(0.5 * m.lik_df) -
                         std::lgamma(0.5 * (m.lik_df + 1.0)));
  } else {
    c.lik_norm = (float)(std::log(std::fabs(m.lik_scale)) + 0.5 * std::log(2.0 * pi));
  }
  c.l_scale = -0.5f * (c.df + 1.0f);
  c.g_scale = (c.df + 1.0f) * c.scale_recp;
  c.prior_recp = (float)(1.0 / m.prior_scale);
  c.prior_norm = (float)(0.5 * std::log(2.0 * pi) + std::log(m.prior_scale));
  c.prior_neg_recp2 = (float)(-1.0 / (m.prior_scale * m.prior_scale));
  return c;
}

int check_model(const bnnhmc_model* m) {
  if (!m) return fail(BNNHMC_ERR_INVALID, "model is null");
  if (!(m->d0 == 22 && m->d1 == 40) && !(m->d0 == 64 && m->d1 == 128))
    return fail(BNNHMC_ERR_INVALID,
                "unsupported layer sizes %d -> %d -> 1 (built: 22 -> 40 -> 1 and 64 -> 128 -> 1)", m->d0,
                m->d1);
  if (m->n <= 0) return fail(BNNHMC_ERR_INVALID, "n must be positive, got %d", m->n);
  if (m->lik_kind != BNNHMC_LIK_STUDENT_T && m->lik_kind != BNNHMC_LIK_GAUSSIAN)
    return fail(BNNHMC_ERR_INVALID, "unknown likelihood kind %d", m->lik_kind);
  if (!(m->lik_scale > 0.0) || !(m->prior_scale > 0.0))
    return fail(BNNHMC_ERR_INVALID, "scales must be positive");
  if (m->lik_kind == BNNHMC_LIK_STUDENT_T && !(m->lik_df > 0.0))
    return fail(BNNHMC_ERR_INVALID, "Student-t degrees of freedom must be positive");
  return BNNHMC_OK;
}

struct DeviceInfo {
  int n_devices = 0;
  int cus = 0;
  std::string arch;
};

int query_device_uncached(DeviceInfo& di) {
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || n <= 0) {
    (void)hipGetLastError();
    return fail(BNNHMC_ERR_NO_DEVICE, "no HIP device visible (%s)",
                e == hipSuccess ? "count is 0" : hipGetErrorString(e));
  }
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, 0));
  di.n_devices = n;
  di.cus = prop.multiProcessorCount;
  di.arch = prop.gcnArchName;
  if (di.arch.rfind("gfx950", 0) != 0)
    return fail(BNNHMC_ERR_NO_DEVICE, "device 0 is %s; this library is built for gfx950 only",
                di.arch.c_str());
  return BNNHMC_OK;
}

// The device is queried once per process; failures are not cached (a later call asks again).
std::mutex g_cache_mutex;
bool g_device_known = false;
DeviceInfo g_device;

int query_device(DeviceInfo& di) {
  std::lock_guard<std::mutex> lock(g_cache_mutex);
  if (!g_device_known) {
    const int rc = query_device_uncached(g_device);
    if (rc) return rc;
    g_device_known = true;
  }
  di = g_device;
  return BNNHMC_OK;
}

// Measurement switch: BNNHMC_PIPELINE=<n> selects the MFMA tile loop of launches that leave `pipeline` at
// its default (and the thread count at 512).  Unset in normal use.
int env_pipeline() {
  const char* e = getenv("BNNHMC_PIPELINE");
  return e && *e ? atoi(e) : 0;
}
// The rows of the windows of a launch are read again at every leapfrog step, and a wave walks its tiles forwards
// in one step and backwards in the next (MfmaHybridLayer), so a step starts with the rows the step before ended
// on: of a batch whose rows are D bytes the 256 MB memory-side cache serves about 256 MB / D, the rest comes from
// HBM (2.3 TB/s at 128 windows of 58368 x 22).  What that traffic costs depends on the card and on the data.  The
// card is power-limited: with the dense operands of the Gaussian benchmark 128 windows at 2 workgroups per chain
// streamed from HBM run at a shader clock of 2.23 GHz on some cards where a cache-resident batch runs at 2.36
// (same cycles per tile), on others they do not lose clock; the reference's Student-t model, whose saturated hidden
// units put zeros into the second contraction, has power to spare everywhere, and then the narrow groups' smaller
// share of exchange time wins.  Evaluations/s of 128 windows at 2 workgroups per chain / 64 at 4 / 32 at 8, every
// CU busy, one card: Gaussian 420 k / 423 k / 413 k, Student-t 428 k / 420 k / 406 k (walking forwards only, the
// Gaussian figures were 416 k / 411 k / 414 k there and 395 k / 396 k / 415 k on a card that loses clock).
// So with the automatic group size a sampler whose chains take turns has two batch shapes -- the largest that
// fits the device, and the largest whose windows' rows fit this budget, 1.4 times the cache (64 windows of that
// size: 344 MB) -- and bnnhmc_run times one launch of each at the start of a call and goes on with the faster.
// BNNHMC_RESIDENT_MB=<n> replaces the budget for measurements (0: no limit, one shape);
// BNNHMC_BATCH_TUNE=0 switches the timing off (the shape within the budget is then used throughout).
size_t resident_row_budget() {
  const char* e = getenv("BNNHMC_RESIDENT_MB");
  const long mb = e && *e ? atol(e) : 358;
  return mb <= 0 ? (size_t)0 : (size_t)mb << 20;
}
// chains of a batch whose windows' rows fit the budget (0: no limit)
int resident_chain_cap(const bnnhmc_model& m, int chains_per_window) {
  const size_t budget = resident_row_budget();
  const size_t window_bytes = (size_t)m.n * (size_t)(m.d0 + 1) * sizeof(float);
  if (budget == 0 || window_bytes > budget) return 0;  // nothing fits anyway: fewest exchanges win
  const size_t windows = budget / window_bytes;
  return (int)std::min<size_t>(windows * (size_t)chains_per_window, (size_t)1 << 20);
}

bool env_batch_tune() {
  const char* e = getenv("BNNHMC_BATCH_TUNE");
  return !(e && *e && atoi(e) == 0);
}

// How a launch is laid over the GPU
struct Plan {
  const void* kernel = nullptr;
  int threads = 0;
  bool wide = false;             // LDS-resident parameter kernel (64 -> 128 -> 1)
  size_t dyn_lds = 0;            // dynamic LDS bytes per workgroup
  size_t wg_scratch_floats = 0;  // private global scratch per workgroup (transitions only)
  int G = 0;
  int wgs_per_cu = 1;
  int max_groups = 0;  // chain groups that can be co-resident at G workgroups each
  int resident_wgs = 0;  // workgroups that can be co-resident on the device
  bool widen = false;    // default group size: a batch that leaves CUs idle gets wider groups
  unsigned spin_limit = 1u << 22;
  int transitions_per_launch = 5;
};

int make_plan_uncached(const bnnhmc_model& m, const bnnhmc_launch* lp, const DeviceInfo& di, Plan& p) {
  bnnhmc_launch l;
  bnnhmc_default_launch(&l);
  if (lp) {
    l.layer = lp->layer;
    if (lp->cus_per_chain > 0) l.cus_per_chain = lp->cus_per_chain;
    if (lp->wgs_per_cu > 0) l.wgs_per_cu = lp->wgs_per_cu;
    if (lp->threads > 0) l.threads = lp->threads;
    if (lp->pipeline > 0) l.pipeline = lp->pipeline;
    if (lp->transitions_per_launch > 0) l.transitions_per_launch = lp->transitions_per_launch;
    if (lp->spin_limit > 0) l.spin_limit = lp->spin_limit;
  }
  if (l.layer != BNNHMC_LAYER_MFMA && l.layer != BNNHMC_LAYER_FFMA)
    return fail(BNNHMC_ERR_INVALID, "unknown layer variant %d", l.layer);
  if (l.wgs_per_cu < 1 || l.wgs_per_cu > 2)
    return fail(BNNHMC_ERR_INVALID, "wgs_per_cu must be 1 or 2, got %d", l.wgs_per_cu);
  // MFMA tile loop: 0 / 4 = prefetched loop with hidden units 32 .. 39 on 4x4 blocks (default), 2 = prefetched
  // loop with three 16-wide hidden tiles, 1 = software-pipelined, 3 = plain
  int loop = 0;
  if (l.layer == BNNHMC_LAYER_MFMA) loop = l.pipeline == 1 ? 1 : (l.pipeline == 3 ? 0 : (l.pipeline == 2 ? 2 : 4));
  // the prefetched loops exist for 512 threads only; other sizes get the plain loop unless a prefetched
  // one was asked for by name (then there is no kernel, reported below)
  if (l.layer == BNNHMC_LAYER_MFMA && l.pipeline == 0 && l.threads > 0 && l.threads != 512) loop = 0;
  p.wide = m.d0 == 64 && m.d1 == 128;
  if (p.wide) {
    if (l.layer != BNNHMC_LAYER_MFMA)
      return fail(BNNHMC_ERR_INVALID, "64 -> 128 -> 1 is built for the MFMA layer only");
    if (l.cus_per_chain > 256)
      return fail(BNNHMC_ERR_INVALID, "64 -> 128 -> 1 supports at most 256 workgroups per chain, got %d",
                  l.cus_per_chain);
    p.threads = l.threads > 0 ? l.threads : 256;
    p.kernel = hmc_kernel_wide_for(m.d0, m.d1, m.lik_kind, p.threads, &p.dyn_lds, &p.wg_scratch_floats);
  } else {
    p.threads = l.threads > 0 ? l.threads
                              : (l.layer == BNNHMC_LAYER_FFMA || l.wgs_per_cu == 2 ? 256 : 512);
    if (l.layer == BNNHMC_LAYER_MFMA && l.pipeline == 0 && p.threads == 512 && env_pipeline() > 0)
      loop = env_pipeline() == 3 ? 0 : env_pipeline();
    p.kernel = hmc_kernel_for(m.d0, m.d1, l.layer, m.lik_kind, p.threads, loop);
  }
  if (!p.kernel)
    return fail(BNNHMC_ERR_INVALID, "no kernel for layer %d with %d threads per workgroup", l.layer,
                p.threads);
  if (p.dyn_lds > 0)
    HIP_TRY(hipFuncSetAttribute(p.kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)p.dyn_lds));
  int per_cu = 0;
  HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, p.kernel, p.threads, p.dyn_lds));
  if (per_cu < 1) return fail(BNNHMC_ERR_RESIDENCY, "kernel does not fit a compute unit");
  p.wgs_per_cu = std::min(per_cu, l.wgs_per_cu);
  const int resident = p.wgs_per_cu * di.cus;
  p.resident_wgs = resident;
  // 0 = automatic.  22 -> 40 -> 1: a batch is the largest power-of-two number of chains that is left
  // and fits (one workgroup per chain at least; a sampler also keeps the rows of a batch within
  // resident_row_budget()), each chain on resident / batch workgroups (measured, evaluations/s with every
  // CU busy: 2 workgroups per chain 419 k, 4: 415 k, 8: 415 k, 16: 382 k, 32: 328 k).  64 -> 128 -> 1: 4
  // workgroups per chain, a last smaller batch widened.
  p.G = l.cus_per_chain > 0 ? l.cus_per_chain : (p.wide ? std::min(4, resident) : 1);
  p.widen = l.cus_per_chain <= 0;
  if (p.G > resident)
    return fail(BNNHMC_ERR_RESIDENCY,
                "%d workgroups per chain requested but only %d can be resident at once", p.G,
                resident);
  p.max_groups = resident / p.G;
  p.spin_limit = l.spin_limit;
  // a launch of the 64 -> 128 -> 1 network does 36 times the work per transition: one transition per
  // launch keeps a kernel's run time in seconds unless the caller asks for more
  p.transitions_per_launch =
      p.wide && !(lp && lp->transitions_per_launch > 0) ? 1 : l.transitions_per_launch;
  return BNNHMC_OK;
}

// Plans are kept per (layer sizes, likelihood, launch parameters): the occupancy query and the
// function-attribute call are made once, so that the step operator touches no device property on
// later calls (the reference's operator does nothing but launch, mcmc_step_ffma.h:395-427).
struct PlanKey {
  int d0, d1, lik, layer, cus_per_chain, wgs_per_cu, threads, pipeline, tpl;
  unsigned spin_limit;
  bool operator==(const PlanKey& o) const {
    return d0 == o.d0 && d1 == o.d1 && lik == o.lik && layer == o.layer &&
           cus_per_chain == o.cus_per_chain && wgs_per_cu == o.wgs_per_cu && threads == o.threads &&
           pipeline == o.pipeline && tpl == o.tpl && spin_limit == o.spin_limit;
  }
};
std::vector<std::pair<PlanKey, Plan>> g_plans;

int make_plan(const bnnhmc_model& m, const bnnhmc_launch* lp, const DeviceInfo& di, Plan& p) {
  bnnhmc_launch l;
  memset(&l, 0, sizeof(l));
  if (lp) l = *lp;
  const PlanKey key{m.d0, m.d1, m.lik_kind, l.layer, l.cus_per_chain, l.wgs_per_cu, l.threads,
                    l.pipeline, l.transitions_per_launch, l.spin_limit};
  {
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    for (const auto& e : g_plans)
      if (e.first == key) {
        p = e.second;
        return BNNHMC_OK;
      }
  }
  const int rc = make_plan_uncached(m, lp, di, p);
  if (rc) return rc;
  std::lock_guard<std::mutex> lock(g_cache_mutex);
  g_plans.emplace_back(key, p);
  return BNNHMC_OK;
}

// Exchange scratch: partial records for `wgs` co-resident workgroups (double-buffered), one totals
// record and one barrier line per chain group (at most `groups`), status words.
// Floats per partial record.  The 64 -> 128 -> 1 kernel exchanges plain floats behind a barrier; the
// 22 -> 40 -> 1 kernel exchanges flagged 8-byte packets (value, step number) that are polled directly.
size_t exchange_slot_floats(int P, bool wide) {
  return (size_t)partial_slot_floats(P) * (wide ? 1 : 2);
}

// Totals records: one per chain group; a 22 -> 40 -> 1 group that reduces by slices (32 workgroups or
// more, so at most wgs / 32 such groups at once) has TOTALS_COPIES of them.
size_t totals_records(int wgs, int groups, bool wide) {
  if (wide) return (size_t)groups;
  return (size_t)std::max(groups, TOTALS_COPIES * std::min(groups, (wgs + 31) / 32));
}

size_t workspace_bytes_for(int P, int wgs, int groups, bool wide) {
  const size_t slot = exchange_slot_floats(P, wide);
  size_t bytes = STATUS_WORDS * sizeof(unsigned);
  bytes += (size_t)(wgs + 31) / 32 * 32 * sizeof(unsigned long long);
  bytes += (size_t)wgs * 2 * slot * sizeof(float);
  bytes += totals_records(wgs, groups, wide) * slot * sizeof(float);
  bytes += (size_t)groups * BARRIER_STRIDE_WORDS * sizeof(unsigned);
  return bytes;
}

// The status words come first and the state hashes right behind them, so that both are found
// without knowing how the rest of the scratch is divided.
struct Workspace {
  unsigned* status;
  unsigned long long* rank_hash;
  float* partials;
  float* totals;
  unsigned* barrier;
  size_t slot_floats;
};
Workspace carve_workspace(void* base, int P, int wgs, int groups, bool wide) {
  Workspace w;
  char* b = (char*)base;
  const size_t slot = exchange_slot_floats(P, wide);
  w.slot_floats = slot;
  w.status = (unsigned*)b;
  b += STATUS_WORDS * sizeof(unsigned);
  w.rank_hash = (unsigned long long*)b;
  b += (size_t)(wgs + 31) / 32 * 32 * sizeof(unsigned long long);
  w.partials = (float*)b;
  b += (size_t)wgs * 2 * slot * sizeof(float);
  w.totals = (float*)b;
  b += totals_records(wgs, groups, wide) * slot * sizeof(float);
  w.barrier = (unsigned*)b;
  return w;
}

// What a launch of `groups` chain groups of G workgroups needs cleared beforehand: the barrier counters
// (64 -> 128 -> 1) or the flags of the packets it will poll (22 -> 40 -> 1: step numbers restart at 1
// with every launch, so no packet of an earlier launch may survive).
hipError_t clear_exchange(const Workspace& w, const KArgs& a, int groups, bool wide, hipStream_t st) {
  if (wide) return launch_fill_u32(w.barrier, (size_t)groups * BARRIER_STRIDE_WORDS, 0u, st);
  hipError_t rc = launch_fill_u32((unsigned*)w.partials, (size_t)groups * 2 * a.G * w.slot_floats, 0u, st);
  if (rc == hipSuccess && a.two_phase)
    rc = launch_fill_u32((unsigned*)w.totals, (size_t)groups * TOTALS_COPIES * w.slot_floats, 0u, st);
  return rc;
}

// Host-side check before every launch: what the kernel of a launch of `groups` chain groups (a.G
// workgroups each, `wgs` in all) will touch in the exchange scratch lies inside the scratch as it was
// carved.  A launch that would not fit is refused, never started.
int check_exchange_bounds(const Workspace& w, const void* base, size_t bytes, const KArgs& a, int groups, int wgs,
                          bool wide) {
  const char* end = (const char*)base + bytes;
  const char* hash_end = (const char*)(w.rank_hash + wgs);
  const char* part_end = (const char*)(w.partials + (size_t)groups * 2 * a.G * w.slot_floats);
  const size_t tot_records = !a.two_phase ? 0 : (size_t)groups * (wide ? 1 : TOTALS_COPIES);
  const char* tot_end = (const char*)(w.totals + tot_records * w.slot_floats);
  const char* bar_end = (const char*)(w.barrier + (wide ? (size_t)groups * BARRIER_STRIDE_WORDS : 0));
  if (hash_end > (const char*)w.partials || part_end > (const char*)w.totals || tot_end > (const char*)w.barrier ||
      bar_end > end || (const char*)w.barrier > end)
    return fail(BNNHMC_ERR_INVALID,
                "internal: a launch of %d chain groups x %d workgroups does not fit the exchange scratch of "
                "%zu bytes; not launched",
                groups, a.G, bytes);
  return BNNHMC_OK;
}

// Synchronises `stream` and reads the status words the launches on it have left since the words
// were last cleared: BNNHMC_ERR_TIMEOUT if a bounded wait expired, BNNHMC_ERR_DIVERGED if the
// workgroups of a chain group did not all hold the same state at the end of a launch.
int read_status(void* workspace, hipStream_t stream) {
  unsigned st[16] = {0};
  HIP_TRY(hipMemcpyAsync(st, workspace, sizeof(st), hipMemcpyDeviceToHost, stream));
  HIP_TRY(hipStreamSynchronize(stream));
  if (st[0] != 0)
    return fail(BNNHMC_ERR_TIMEOUT,
                "a workgroup (%u) waited longer than the spin limit for its chain group; the launch "
                "was abandoned",
                st[1] ? st[1] - 1 : 0u);
  if (st[4] != 0)
    return fail(BNNHMC_ERR_DIVERGED,
                "workgroup %u (chain group %u of its launch) integrated a different state than the first "
                "workgroup of its group (state hash %08x%08x vs %08x%08x): a partial record was read before "
                "it was complete",
                st[4] - 1, st[5], st[7], st[6], st[9], st[8]);
  return BNNHMC_OK;
}

// Chains of the next batch when `left` are still to run: as many as fit; with the automatic group size
// of the 22 -> 40 -> 1 kernel the largest power of two of them, so that the batch fills the device with
// equal groups (see make_plan_uncached).
int batch_size(const Plan& p, int left, int limit = 0) {
  int groups = std::min(p.max_groups, left);
  if (limit > 0) groups = std::min(groups, limit);
  if (p.widen && !p.wide) {
    int b = 1;
    while (b * 2 <= groups) b *= 2;
    groups = b;
  }
  return groups;
}

// Workgroups per chain for a batch of `groups` chains: the configured count, widened by powers of
// two while the whole batch still fits the device (a last, smaller batch then uses every CU).
int widen_group(int G, int groups, int resident_wgs, int cap) {
  while (G * 2 * groups <= resident_wgs && G * 2 <= cap) G *= 2;
  return G;
}

void set_grid(KArgs& a, int groups, int G, bool wide, int* workgroups) {
  const int wgs = groups * G;
  a.G = G;
  // From 32 workgroups per chain on, the first workgroups of a group each reduce one slice of the
  // records (32 parameters, 31 reducers; from 64 workgroups on 16 parameters, 61 reducers) and everyone
  // reads the totals, instead of everyone reading every record.  Measured on
  // MI355X with the 22 -> 40 -> 1 kernel (evaluations/s, all-read vs slices): G = 32: 278 k vs 288 k,
  // G = 64: 183 k vs 230 k.  The 64 -> 128 -> 1 kernel, whose hand-offs go through barriers, switches
  // above 64.
  a.two_phase = G >= (wide ? 65 : 32) ? 1 : 0;
  a.n_groups = groups;
  a.xcd_map = (wgs % 8 == 0) && ((wgs / 8) % G == 0) ? 1 : 0;
  *workgroups = wgs;
}

// Test hook: BNNHMC_DEBUG_DROP_ARRIVAL=<rank> makes that rank of every chain group withhold its
// arrival at the group barrier, so that the bounded wait of the others expires (every workgroup still
// exits normally).  Unset in normal use.
int debug_drop_rank() {
  const char* e = getenv("BNNHMC_DEBUG_DROP_ARRIVAL");
  return e && *e ? atoi(e) : -1;
}

// Measurement switch: BNNHMC_BALANCE=0 turns off the pacing of the two waves that share a SIMD (wave
// priorities in the prefetched tile loop).  Unset in normal use (pacing on).
int env_balance() {
  const char* e = getenv("BNNHMC_BALANCE");
  return e && *e ? atoi(e) : 1;
}
// Test hook: BNNHMC_DEBUG_PERTURB_HASH=<rank> makes that rank of every chain group flip one bit of
// the state hash it reports (its memory traffic and its results are untouched), so that the
// comparison of the hashes fails.  Unset in normal use.
int debug_perturb_hash_rank() {
  const char* e = getenv("BNNHMC_DEBUG_PERTURB_HASH");
  return e && *e ? atoi(e) : -1;
}

// host restatement of the hidden activation (kernel_helpers.h:34-42) for the data generator
inline float host_tanh(float x) {
  const float e = exp2f(x * -2.88539008177792681472f);
  const float sigm = 1.0f / (1.0f + e);
  return std::fabs(x) < 0.0048176045529544353485f ? x : fmaf(sigm, 2.0f, -1.0f);
}

void generate_rows(uint32_t seed, uint32_t window, int row_begin, int row_end, int d0, int d1,
                   float noise_sigma, const std::vector<float>& th, float* X, float* y) {
  const Layout L = make_layout(d0, d1);
  std::vector<float> h(d1);
  for (int i = row_begin; i < row_end; ++i) {
    float* x = X + (size_t)i * d0;
    for (int k = 0; k < d0; ++k) x[k] = rng_normal(seed, window, STREAM_X, 0, (uint64_t)i * d0 + k);
    for (int c = 0; c < d1; ++c) h[c] = th[L.ob1 + c];
    for (int k = 0; k < d0; ++k)
      for (int c = 0; c < d1; ++c) h[c] = fmaf(th[(size_t)k * d1 + c], x[k], h[c]);
    float yh = th[L.ob2];
    for (int c = 0; c < d1; ++c) yh = fmaf(th[L.ow2 + c], host_tanh(h[c]), yh);
    y[i] = fmaf(noise_sigma, rng_normal(seed, window, STREAM_NOISE, 0, (uint64_t)i), yh);
  }
}

// Every element is a function of (seed, window, its index) alone, so the rows can be filled by any
// number of threads with the same result.
void generate_window_host(uint32_t seed, uint32_t window, int n, int d0, int d1, float teacher_scale,
                          float noise_sigma, float* X, float* y, float* teacher) {
  const Layout L = make_layout(d0, d1);
  std::vector<float> th(L.P);
  for (int p = 0; p < L.P; ++p)
    th[p] = teacher_scale * rng_normal(seed, window, STREAM_TEACHER, 0, (uint64_t)p);
  if (teacher) memcpy(teacher, th.data(), sizeof(float) * L.P);
  unsigned hw = std::thread::hardware_concurrency();
  const int n_threads = (int)std::max(1u, std::min({hw ? hw : 1u, 16u, (unsigned)(n / 4096 + 1)}));
  if (n_threads == 1) {
    generate_rows(seed, window, 0, n, d0, d1, noise_sigma, th, X, y);
    return;
  }
  std::vector<std::thread> pool;
  for (int t = 0; t < n_threads; ++t) {
    const int b = (int)((long)n * t / n_threads), e = (int)((long)n * (t + 1) / n_threads);
    pool.emplace_back(generate_rows, seed, window, b, e, d0, d1, noise_sigma, std::cref(th), X, y);
  }
  for (auto& t : pool) t.join();
}

}  // namespace

// Result slots of bnnhmc_get_loss_values: a static device array (every GPU holds its own copy), whose
// address on the current device is looked up once per device.
constexpr int LOSS_SLOTS = 64;
constexpr int MAX_DEVICES = 16;
static __device__ __align__(256) float g_loss_slots[LOSS_SLOTS][2];

// Exchange scratch of bnnhmc_mcmc_step_static: partial-gradient records, barrier and status words of
// one step operator call at a time per GPU.  4.5 MiB covers one chain on 256 workgroups for
// 22 -> 40 -> 1 and on up to 64 workgroups for 64 -> 128 -> 1 (wider groups of that network need more and
// are refused).  Every GPU the library runs on
// holds its own copy until the process ends; host code reaches it only through the address looked up
// once per device below (the array's name is a host-side stand-in, not a device address).
constexpr size_t STEP_SCRATCH_BYTES = 4608u * 1024u;
static __device__ __align__(256) unsigned char g_step_scratch[STEP_SCRATCH_BYTES];

namespace {
void* g_step_scratch_ptr[MAX_DEVICES] = {nullptr};

int step_scratch(void** out) {
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= MAX_DEVICES)
    return fail(BNNHMC_ERR_INVALID, "device index %d is beyond the %d this library keeps state for", dev,
                MAX_DEVICES);
  std::lock_guard<std::mutex> lock(g_cache_mutex);
  if (!g_step_scratch_ptr[dev]) {
    void* p = nullptr;
    HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(g_step_scratch)));
    g_step_scratch_ptr[dev] = p;
  }
  *out = g_step_scratch_ptr[dev];
  return BNNHMC_OK;
}

float* g_loss_slots_ptr[MAX_DEVICES] = {nullptr};
unsigned g_loss_next = 0;

int loss_slot(float** out) {
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= MAX_DEVICES)
    return fail(BNNHMC_ERR_INVALID, "device index %d is beyond the %d this library keeps state for", dev,
                MAX_DEVICES);
  std::lock_guard<std::mutex> lock(g_cache_mutex);
  if (!g_loss_slots_ptr[dev]) {
    void* p = nullptr;
    HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(g_loss_slots)));
    g_loss_slots_ptr[dev] = (float*)p;
  }
  *out = g_loss_slots_ptr[dev] + 2 * (size_t)(g_loss_next++ % LOSS_SLOTS);
  return BNNHMC_OK;
}
}  // namespace

// =================================================================================================
struct bnnhmc_sampler {
  bnnhmc_model model;
  bnnhmc_hmc hmc;
  DeviceInfo dev;
  Plan plan;
  Layout L;
  ModelConsts mc;
  int n_windows = 0, cpw = 0, n_chains = 0;
  int n_pad = 0;       // rows rounded up to 16
  int st_stride = 0;   // floats per chain state record
  int trace_len = 0;
  bool data_set = false, inited = false;
  std::vector<char> window_set;
  hipStream_t stream = nullptr;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  hipEvent_t ev_t0 = nullptr, ev_t1 = nullptr;  // around one launch while the batch shape is being chosen
  int batch_cap = 0;        // chains of a batch whose windows' rows fit resident_row_budget() (0: no such limit)
  int batch_limit = 0;      // the limit bnnhmc_run applies at present: batch_cap or 0 (what fits the device)
  double tuned_rate[2] = {0.0, 0.0};  // evaluations per ms of the last trial launches: within the budget, device-wide
  long quanta_since_tune = -1;        // quanta dealt since the shapes were last timed (-1: never)
  // device memory
  float* X = nullptr;
  float* y = nullptr;
  float* st_w = nullptr;
  float* st_g = nullptr;
  float* st_eps = nullptr;
  int* st_t = nullptr;
  int* st_sel = nullptr;
  int* st_nacc = nullptr;
  float* ell0 = nullptr;
  float* ell1 = nullptr;
  float* samples = nullptr;
  float* tr_la = nullptr;
  int* tr_acc = nullptr;
  float* tr_eps = nullptr;
  void* workspace = nullptr;
  size_t workspace_bytes = 0;
  float* wg_scratch = nullptr;  // wide-layer kernel: per-workgroup accepted state and start momentum
  float* tmp = nullptr;       // evaluation scratch: w | grad | prior (3 * st_stride) ...
  float* tmp_ell = nullptr;   // ... and n_pad rows
  double* tmp_sums = nullptr; // [max_groups][2]
  unsigned long long* debug_phase = nullptr;  // set when BNNHMC_DEBUG_PHASE is in the environment
  // timing
  double kernel_ms = 0.0;
  long launches = 0, grad_evals = 0;
  int last_workgroups = 0;
  int transitions_done = 0;

  std::vector<void*> allocs;
  template <typename T>
  int alloc(T** p, size_t count) {
    void* q = nullptr;
    hipError_t e = hipMalloc(&q, std::max<size_t>(count, 1) * sizeof(T));
    if (e != hipSuccess)
      return fail(BNNHMC_ERR_HIP, "hipMalloc of %zu bytes failed: %s", count * sizeof(T),
                  hipGetErrorString(e));
    allocs.push_back(q);
    *p = (T*)q;
    return BNNHMC_OK;
  }
};

namespace {

KArgs base_args(const bnnhmc_sampler* s) {
  KArgs a;
  memset(&a, 0, sizeof(a));
  a.n = s->model.n;
  a.n_tiles = (s->model.n + 15) / 16;
  a.mc = s->mc;
  a.X = s->X;
  a.y = s->y;
  a.x_stride = (long)s->model.n * s->model.d0;
  a.y_stride = s->n_pad;
  a.x_vec_ok = (s->model.d0 % 2 == 0) ? 1 : 0;  // hipMalloc alignment, even row length
  a.y_vec_ok = 1;                               // window stride is a multiple of 16 rows
  a.chains_per_window = s->cpw;
  a.fixed_window = -1;
  a.L = s->hmc.leapfrog_steps;
  a.spin_limit = s->plan.spin_limit;
  a.debug_drop_rank = debug_drop_rank();
  a.debug_perturb_hash_rank = debug_perturb_hash_rank();
  a.balance = env_balance();
  Workspace w = carve_workspace(s->workspace, s->L.P, s->plan.resident_wgs, s->plan.max_groups, s->plan.wide);
  a.partials = w.partials;
  a.totals = w.totals;
  a.barrier = w.barrier;
  a.status = w.status;
  a.rank_hash = w.rank_hash;
  a.wg_scratch = s->wg_scratch;
  return a;
}

int launch_and_count(bnnhmc_sampler* s, KArgs& a, int groups) {
  int wgs = 0;
  set_grid(a, groups, s->plan.widen ? widen_group(s->plan.G, groups, s->plan.resident_wgs, 256) : s->plan.G,
           s->plan.wide, &wgs);
  const Workspace w = carve_workspace(s->workspace, s->L.P, s->plan.resident_wgs, s->plan.max_groups, s->plan.wide);
  const int fits = check_exchange_bounds(w, s->workspace, s->workspace_bytes, a, groups, wgs, s->plan.wide);
  if (fits != BNNHMC_OK) return fits;
  HIP_TRY(clear_exchange(w, a, groups, s->plan.wide, s->stream));
  HIP_TRY(launch_hmc_kernel(s->plan.kernel, a, wgs, s->plan.threads, s->plan.dyn_lds, s->stream));
  HIP_TRY(launch_compare_hashes(a.rank_hash, wgs, a.G, a.status, s->stream));
  s->last_workgroups = wgs;
  return BNNHMC_OK;
}

int check_status(bnnhmc_sampler* s) {
  const int rc = read_status(s->workspace, s->stream);
  if (rc == BNNHMC_ERR_TIMEOUT || rc == BNNHMC_ERR_DIVERGED) {
    // the words are sticky until cleared: the sampler stays usable after the error is reported
    const std::string msg = g_last_error;
    HIP_TRY(launch_fill_u32((unsigned*)s->workspace, STATUS_WORDS, 0u, s->stream));
    HIP_TRY(hipStreamSynchronize(s->stream));
    g_last_error = msg;
  }
  return rc;
}

// evaluate MODE_STEPS with L = 1, eps = 0 for `groups` parameter vectors starting at w_dev
int eval_groups(bnnhmc_sampler* s, int window, const float* w_dev, long in_stride, int groups,
                float* g_out, float* prior_out, long out_stride, float* ell_out, long ell_stride,
                double* sums_out) {
  KArgs a = base_args(s);
  a.mode = MODE_STEPS;
  a.L = 1;
  a.eps_in = 0.0f;
  a.fixed_window = window;
  a.chain_base = 0;
  a.w_in = w_dev;
  a.in_stride = in_stride;
  a.g_out = g_out;
  a.prior_out = prior_out;
  a.out_stride = out_stride;
  a.ell_out = ell_out;
  a.ell_stride = ell_stride;
  a.sums_out = sums_out;
  return launch_and_count(s, a, groups);
}

}  // namespace

extern "C" {

void bnnhmc_default_model(bnnhmc_model* m) {
  if (!m) return;
  m->d0 = 22;
  m->d1 = 40;
  m->n = 58368;
  m->lik_kind = BNNHMC_LIK_STUDENT_T;
  m->lik_scale = 100.0;
  m->lik_df = 2.2;
  m->prior_scale = 200.0;
}

void bnnhmc_default_hmc(bnnhmc_hmc* h) {
  if (!h) return;
  h->leapfrog_steps = 1000;
  h->burn_in = 100;
  h->n_samples = 800;
  h->adapt_steps = 100;
  h->eps0 = 0.01f;
  h->target_rate = 0.2f;
  h->decrement = 0.1f;
  h->increment = 0.01f;
  h->seed = 0;
  h->chain_id_base = 0;
}

void bnnhmc_default_launch(bnnhmc_launch* l) {
  if (!l) return;
  l->layer = BNNHMC_LAYER_MFMA;
  l->cus_per_chain = 0;
  l->wgs_per_cu = 1;
  l->threads = 0;
  l->pipeline = 0;
  l->transitions_per_launch = 5;
  l->spin_limit = 1u << 22;
}

int bnnhmc_num_params(int d0, int d1) { return make_layout(d0, d1).P; }

const char* bnnhmc_last_error(void) { return g_last_error.c_str(); }

int bnnhmc_device_info(int* n_devices, int* compute_units, char* arch, size_t arch_len) {
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    n = 0;
  }
  if (n_devices) *n_devices = n;
  if (compute_units) *compute_units = 0;
  if (arch && arch_len) arch[0] = 0;
  if (n <= 0) return fail(BNNHMC_ERR_NO_DEVICE, "no HIP device visible");
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, 0));
  if (compute_units) *compute_units = prop.multiProcessorCount;
  if (arch && arch_len) {
    strncpy(arch, prop.gcnArchName, arch_len - 1);
    arch[arch_len - 1] = 0;
  }
  return BNNHMC_OK;
}

int bnnhmc_generate_window_host(uint32_t seed, uint32_t window, int n, int d0, int d1,
                                float teacher_scale, float noise_sigma, float* x_out, float* y_out,
                                float* teacher_out) {
  if (n < 0 || d0 <= 0 || d1 <= 0 || !x_out || !y_out)
    return fail(BNNHMC_ERR_INVALID, "bad arguments to bnnhmc_generate_window_host");
  generate_window_host(seed, window, n, d0, d1, teacher_scale, noise_sigma, x_out, y_out,
                       teacher_out);
  return BNNHMC_OK;
}

int bnnhmc_read_reference_data(const char* path, int n, int d0, int total_cols, int skip_cols,
                               float* x_out, float* y_out) {
  if (!path || n < 0 || d0 <= 0 || skip_cols < 0 || total_cols < skip_cols + 1 + d0 || !x_out || !y_out)
    return fail(BNNHMC_ERR_INVALID, "bad arguments to bnnhmc_read_reference_data");
  FILE* fp = std::fopen(path, "r");
  if (!fp) return fail(BNNHMC_ERR_INVALID, "failed to read file '%s'", path);
  char buf[256];
  // the first line is a header of total_cols names (io.h:60-62)
  for (int j = 0; j < total_cols; ++j)
    if (std::fscanf(fp, "%255s", buf) != 1) break;
  for (int i = 0; i < n; ++i) {
    for (int j = 0; j < total_cols; ++j) {
      if (std::fscanf(fp, "%255s", buf) != 1) {
        std::fclose(fp);
        return fail(BNNHMC_ERR_INVALID, "'%s' ends at row %d, column %d (expected %d rows of %d columns)",
                    path, i, j, n, total_cols);
      }
      if (j < skip_cols || j > skip_cols + d0) continue;  // io.h:65-69
      char* end = nullptr;
      const float v = std::strtof(buf, &end);
      if (end == buf) {
        std::fclose(fp);
        return fail(BNNHMC_ERR_INVALID, "'%s' row %d column %d is not a number: '%s'", path, i, j, buf);
      }
      if (j == skip_cols) y_out[i] = v;                       // io.h:71-76
      else x_out[(size_t)i * d0 + (j - skip_cols - 1)] = v;   // io.h:77
    }
  }
  std::fclose(fp);
  return BNNHMC_OK;
}

// ---- host mirrors of the RNG, for callers that need the streams on the CPU ----
uint32_t bnnhmc_rng_word(uint32_t seed, uint32_t id, uint32_t stream, uint32_t t, uint64_t index) {
  return rng_word(seed, id, stream, t, index);
}
float bnnhmc_rng_normal(uint32_t seed, uint32_t id, uint32_t stream, uint32_t t, uint64_t index) {
  return rng_normal(seed, id, stream, t, index);
}
float bnnhmc_rng_log_uniform(uint32_t seed, uint32_t chain_id, uint32_t t) {
  return rng_log_uniform(seed, chain_id, t);
}

// =================================================================================================
// operator level
// =================================================================================================
// workgroups the step operator gives its single chain: the configured count, or by default the
// largest power of two that is resident at once (at most 256)
static int step_group(const bnnhmc_launch* launch, int resident_wgs, int cap) {
  if (launch && launch->cus_per_chain > 0) return launch->cus_per_chain;
  int G = 1;
  while (G * 2 <= resident_wgs && G * 2 <= cap) G *= 2;
  return G;
}

size_t bnnhmc_step_workspace_bytes(const bnnhmc_model* model, const bnnhmc_launch* launch) {
  if (!model) return 0;
  // sized for the default group (256) when none is configured, whatever device is present
  const int G = launch && launch->cus_per_chain > 0 ? launch->cus_per_chain : 256;
  return workspace_bytes_for(make_layout(model->d0, model->d1).P, G, 1, model->d0 == 64 && model->d1 == 128);
}

int bnnhmc_step_launch_info(const bnnhmc_model* model, const bnnhmc_launch* launch, int* workgroups,
                            int* threads, int* rows_per_wave, size_t* lds_bytes, size_t* lds_max_bytes) {
  int rc = check_model(model);
  if (rc) return rc;
  DeviceInfo di;
  rc = query_device(di);
  if (rc) return rc;
  Plan plan;
  rc = make_plan(*model, launch, di, plan);
  if (rc) return rc;
  const int G = step_group(launch, plan.resident_wgs, 256);
  const int waves = G * (plan.threads / 64), tiles = (model->n + 15) / 16;
  if (workgroups) *workgroups = G;
  if (threads) *threads = plan.threads;
  if (rows_per_wave) *rows_per_wave = 16 * ((tiles + waves - 1) / waves);
  if (lds_bytes || lds_max_bytes) {
    hipFuncAttributes attr;
    HIP_TRY(hipFuncGetAttributes(&attr, plan.kernel));
    if (lds_bytes) *lds_bytes = attr.sharedSizeBytes + plan.dyn_lds;
    if (lds_max_bytes) {
      int v = 0;
      HIP_TRY(hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, 0));
      *lds_max_bytes = (size_t)v;
    }
  }
  return BNNHMC_OK;
}

// The step operator on a given exchange scratch; allocates nothing (device and plan queries happen on
// the first call for a configuration only, and allocate nothing either).
static int mcmc_step_on(const bnnhmc_model* model, const bnnhmc_launch* launch, const float* x,
                        const float* y, const float* weights_prev, float* weights_next,
                        const float* mom_prev, float* mom_next, const float* grad_prev,
                        float* grad_cur, float* grad_next, float* loss_values, void* workspace,
                        size_t workspace_bytes, float eps, int lp_steps, void* stream) {
  int rc = check_model(model);
  if (rc) return rc;
  if (!x || !y || !weights_prev || !weights_next || !mom_prev || !mom_next || !grad_prev ||
      !grad_cur || !loss_values || !workspace)
    return fail(BNNHMC_ERR_INVALID, "null device pointer passed to bnnhmc_mcmc_step");
  if (lp_steps < 1) return fail(BNNHMC_ERR_INVALID, "lp_steps must be >= 1, got %d", lp_steps);
  if ((uintptr_t)workspace % 16 != 0)
    return fail(BNNHMC_ERR_INVALID, "workspace must be 16-byte aligned");
  DeviceInfo di;
  rc = query_device(di);
  if (rc) return rc;
  Plan plan;
  rc = make_plan(*model, launch, di, plan);
  if (rc) return rc;
  const Layout L = make_layout(model->d0, model->d1);
  const int G = step_group(launch, plan.resident_wgs, 256);
  if (G > plan.resident_wgs)
    return fail(BNNHMC_ERR_RESIDENCY, "%d workgroups per chain requested but only %d can be resident", G,
                plan.resident_wgs);
  if (workspace_bytes < workspace_bytes_for(L.P, G, 1, plan.wide))
    return fail(BNNHMC_ERR_INVALID, "workspace too small: %zu < %zu bytes", workspace_bytes,
                workspace_bytes_for(L.P, G, 1, plan.wide));
  hipStream_t st = (hipStream_t)stream;
  KArgs a;
  memset(&a, 0, sizeof(a));
  a.n = model->n;
  a.n_tiles = (model->n + 15) / 16;
  a.mc = make_consts(*model);
  a.X = x;
  a.y = y;
  // vector loads of the rows: 8 bytes (22 -> 40) or 16 bytes (64 -> 128)
  a.x_vec_ok = ((uintptr_t)x % (plan.wide ? 16 : 8) == 0 && model->d0 % 2 == 0) ? 1 : 0;
  a.y_vec_ok = ((uintptr_t)y % 16 == 0) ? 1 : 0;
  a.chains_per_window = 1;
  a.fixed_window = 0;
  a.mode = MODE_STEPS;
  a.L = lp_steps;
  a.eps_in = eps;
  a.w_in = weights_prev;
  a.m_in = mom_prev;
  a.g_in = grad_prev;
  a.w_out = weights_next;
  a.m_out = mom_next;
  a.g_out = grad_cur;
  a.g_zero = grad_next;
  a.ell_out = loss_values;
  a.prior_out = loss_values + model->n;
  a.spin_limit = plan.spin_limit;
  a.debug_drop_rank = debug_drop_rank();
  a.debug_perturb_hash_rank = debug_perturb_hash_rank();
  a.balance = env_balance();
  Workspace w = carve_workspace(workspace, L.P, G, 1, plan.wide);
  a.partials = w.partials;
  a.totals = w.totals;
  a.barrier = w.barrier;
  a.status = w.status;
  a.rank_hash = w.rank_hash;
  int wgs = 0;
  set_grid(a, 1, G, plan.wide, &wgs);
  const int fits = check_exchange_bounds(w, workspace, workspace_bytes, a, 1, wgs, plan.wide);
  if (fits != BNNHMC_OK) return fits;
  // The exchange area starts from zero on every call.  The status words are cleared on the first use
  // of a workspace only: the record of a step that failed stays until bnnhmc_step_check reports it.
  HIP_TRY(launch_prepare_status(w.status, st));
  HIP_TRY(clear_exchange(w, a, 1, plan.wide, st));
  HIP_TRY(launch_hmc_kernel(plan.kernel, a, wgs, plan.threads, plan.dyn_lds, st));
  HIP_TRY(launch_compare_hashes(a.rank_hash, wgs, G, a.status, st));
  return BNNHMC_OK;
}

int bnnhmc_mcmc_step(const bnnhmc_model* model, const bnnhmc_launch* launch, const float* x,
                     const float* y, const float* weights_prev, float* weights_next,
                     const float* mom_prev, float* mom_next, const float* grad_prev,
                     float* grad_cur, float* grad_next, float* loss_values, void* workspace,
                     size_t workspace_bytes, float eps, int lp_steps, void* stream) {
  return mcmc_step_on(model, launch, x, y, weights_prev, weights_next, mom_prev, mom_next, grad_prev,
                      grad_cur, grad_next, loss_values, workspace, workspace_bytes, eps, lp_steps, stream);
}

int bnnhmc_mcmc_step_static(const bnnhmc_model* model, const bnnhmc_launch* launch, const float* x,
                            const float* y, const float* weights_prev, float* weights_next,
                            const float* mom_prev, float* mom_next, const float* grad_prev,
                            float* grad_cur, float* grad_next, float* loss_values, float eps,
                            int lp_steps, void* stream) {
  if (!model) return fail(BNNHMC_ERR_INVALID, "model is null");
  const size_t need = bnnhmc_step_workspace_bytes(model, launch);
  if (need > STEP_SCRATCH_BYTES)
    return fail(BNNHMC_ERR_INVALID,
                "this configuration needs %zu bytes of exchange scratch; bnnhmc_mcmc_step_static holds %zu "
                "(use bnnhmc_mcmc_step with a workspace of your own)",
                need, (size_t)STEP_SCRATCH_BYTES);
  void* scratch = nullptr;
  const int rc = step_scratch(&scratch);
  if (rc) return rc;
  return mcmc_step_on(model, launch, x, y, weights_prev, weights_next, mom_prev, mom_next, grad_prev,
                      grad_cur, grad_next, loss_values, scratch, STEP_SCRATCH_BYTES, eps, lp_steps, stream);
}

int bnnhmc_step_check(const bnnhmc_model* model, const bnnhmc_launch* launch, void* workspace,
                      void* stream) {
  (void)launch;
  if (!model) return fail(BNNHMC_ERR_INVALID, "null argument to bnnhmc_step_check");
  if (!workspace) {  // the step ran on the library's own scratch (bnnhmc_mcmc_step_static)
    const int rc = step_scratch(&workspace);
    if (rc) return rc;
  }
  // the status words sit at the start of the workspace whatever the launch parameters were
  const int rc = read_status(workspace, (hipStream_t)stream);
  if (rc == BNNHMC_ERR_TIMEOUT || rc == BNNHMC_ERR_DIVERGED) {
    // reported once: the record is cleared so that the workspace can be used again
    const std::string msg = g_last_error;
    HIP_TRY(launch_clear_status((unsigned*)workspace, (hipStream_t)stream));
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    g_last_error = msg;
  }
  return rc;
}

int bnnhmc_sample_momentum(uint32_t seed, uint32_t chain_id, uint32_t transition, int n,
                           float* prev_lp_mom, float* mom_next, void* stream) {
  if (n < 0 || (n > 0 && !prev_lp_mom && !mom_next))
    return fail(BNNHMC_ERR_INVALID, "bad arguments to bnnhmc_sample_momentum");
  HIP_TRY(launch_sample_momentum(seed, chain_id, transition, n, prev_lp_mom, mom_next,
                                 (hipStream_t)stream));
  return BNNHMC_OK;
}

int bnnhmc_log_acpt(int n_loss, int n_mom, const float* prev_loss, const float* new_loss,
                    const float* prev_mom, const float* new_mom, const float* grad_cur, float eps,
                    float* log_acpt_out, float* host_out, void* stream) {
  if (n_loss < 0 || n_mom < 0 || (n_loss > 0 && (!prev_loss || !new_loss)) ||
      (n_mom > 0 && (!prev_mom || !new_mom || !grad_cur)))
    return fail(BNNHMC_ERR_INVALID, "bad arguments to bnnhmc_log_acpt");
  if (!log_acpt_out) return fail(BNNHMC_ERR_INVALID, "log_acpt_out (device) must not be null");
  hipStream_t st = (hipStream_t)stream;
  HIP_TRY(launch_log_acpt(n_loss, n_mom, prev_loss, new_loss, prev_mom, new_mom, grad_cur, eps,
                          log_acpt_out, st));
  if (host_out) {
    HIP_TRY(hipMemcpyAsync(host_out, log_acpt_out, sizeof(float), hipMemcpyDeviceToHost, st));
    HIP_TRY(hipStreamSynchronize(st));
  }
  return BNNHMC_OK;
}

int bnnhmc_get_loss_values(const float* loss_values, int n, int n_params, float* loss1_host,
                           float* loss2_host, void* stream) {
  if (!loss_values || n < 0 || n_params < 0)
    return fail(BNNHMC_ERR_INVALID, "bad arguments to bnnhmc_get_loss_values");
  hipStream_t st = (hipStream_t)stream;
  // No allocation (the reference allocates its reduction scratch once, kernel_helpers.h:194-204):
  // the two sums land in one of LOSS_SLOTS pairs of a static device array, handed out round-robin; a
  // pair is in use only until this call returns, so up to LOSS_SLOTS calls may overlap.
  float* d = nullptr;
  int rc = loss_slot(&d);
  if (rc) return rc;
  HIP_TRY(launch_loss_sums(loss_values, n, n_params, d, st));
  float h[2] = {0, 0};
  HIP_TRY(hipMemcpyAsync(h, d, sizeof(h), hipMemcpyDeviceToHost, st));
  HIP_TRY(hipStreamSynchronize(st));
  if (loss1_host) *loss1_host = h[0];
  if (loss2_host) *loss2_host = h[1];
  return BNNHMC_OK;
}

// =================================================================================================
// sampler level
// =================================================================================================
int bnnhmc_create(const bnnhmc_model* model, const bnnhmc_hmc* hmc, const bnnhmc_launch* launch,
                  int n_windows, int chains_per_window, bnnhmc_sampler** out) {
  if (!out) return fail(BNNHMC_ERR_INVALID, "out is null");
  *out = nullptr;
  int rc = check_model(model);
  if (rc) return rc;
  if (!hmc) return fail(BNNHMC_ERR_INVALID, "hmc is null");
  if (hmc->leapfrog_steps < 1 || hmc->burn_in < 0 || hmc->n_samples < 0 || hmc->adapt_steps < 0)
    return fail(BNNHMC_ERR_INVALID, "bad sampler constants");
  if (n_windows < 1 || chains_per_window < 1)
    return fail(BNNHMC_ERR_INVALID, "n_windows and chains_per_window must be >= 1");
  {
    // the exchange numbers the leapfrog steps of a launch in 32 bits, from 1 (0 = the cleared state)
    bnnhmc_launch dl;
    bnnhmc_default_launch(&dl);
    const long long tpl = launch && launch->transitions_per_launch > 0 ? launch->transitions_per_launch
                                                                         : dl.transitions_per_launch;
    if (tpl * (long long)hmc->leapfrog_steps >= 0xFFFFFFFFll)
      return fail(BNNHMC_ERR_INVALID,
                  "transitions_per_launch (%lld) x leapfrog_steps (%d) must stay below 2^32 - 1", tpl,
                  hmc->leapfrog_steps);
  }
  DeviceInfo di;
  rc = query_device(di);
  if (rc) return rc;
  bnnhmc_sampler* s = new (std::nothrow) bnnhmc_sampler();
  if (!s) return fail(BNNHMC_ERR_INVALID, "out of host memory");
  s->model = *model;
  s->hmc = *hmc;
  s->dev = di;
  s->L = make_layout(model->d0, model->d1);
  s->mc = make_consts(*model);
  s->n_windows = n_windows;
  s->cpw = chains_per_window;
  s->n_chains = n_windows * chains_per_window;
  s->n_pad = (model->n + 15) / 16 * 16;
  s->st_stride = (s->L.P + 3) / 4 * 4;
  s->trace_len = hmc->burn_in + hmc->n_samples;
  s->window_set.assign(n_windows, 0);
  rc = make_plan(*model, launch, di, s->plan);
  if (rc) {
    delete s;
    return rc;
  }
  if (s->plan.widen && !s->plan.wide) {
    const int cap = resident_chain_cap(*model, chains_per_window);
    if (cap > 0 && cap < s->plan.max_groups) s->batch_cap = s->batch_limit = cap;
  }
  auto bail = [&](int code) {
    bnnhmc_destroy(s);
    return code;
  };
  hipError_t e = hipStreamCreate(&s->stream);
  if (e == hipSuccess) e = hipEventCreate(&s->ev0);
  if (e == hipSuccess) e = hipEventCreate(&s->ev1);
  if (e == hipSuccess) e = hipEventCreate(&s->ev_t0);
  if (e == hipSuccess) e = hipEventCreate(&s->ev_t1);
  if (e != hipSuccess) {
    fail(BNNHMC_ERR_HIP, "stream/event creation failed: %s", hipGetErrorString(e));
    return bail(BNNHMC_ERR_HIP);
  }
  const size_t C = s->n_chains;
  const int eval_groups_max = s->plan.max_groups;
  s->workspace_bytes = workspace_bytes_for(s->L.P, s->plan.resident_wgs, s->plan.max_groups, s->plan.wide);
  char* ws = nullptr;
  if ((rc = s->alloc(&s->X, (size_t)n_windows * model->n * model->d0)) ||
      (rc = s->alloc(&s->y, (size_t)n_windows * s->n_pad)) ||
      (rc = s->alloc(&s->st_w, C * s->st_stride)) || (rc = s->alloc(&s->st_g, C * s->st_stride)) ||
      (rc = s->alloc(&s->st_eps, C)) || (rc = s->alloc(&s->st_t, C)) ||
      (rc = s->alloc(&s->st_sel, C)) || (rc = s->alloc(&s->st_nacc, C)) ||
      (rc = s->alloc(&s->ell0, C * s->n_pad)) || (rc = s->alloc(&s->ell1, C * s->n_pad)) ||
      (rc = s->alloc(&s->samples, C * (size_t)hmc->n_samples * s->L.P)) ||
      (rc = s->alloc(&s->tr_la, C * s->trace_len)) || (rc = s->alloc(&s->tr_acc, C * s->trace_len)) ||
      (rc = s->alloc(&s->tr_eps, C * s->trace_len)) || (rc = s->alloc(&ws, s->workspace_bytes)) ||
      (rc = s->alloc(&s->tmp, (size_t)3 * s->st_stride * eval_groups_max)) ||
      (rc = s->alloc(&s->tmp_ell, (size_t)s->n_pad)) ||
      (rc = s->alloc(&s->tmp_sums, (size_t)2 * eval_groups_max)) ||
      (rc = s->alloc(&s->wg_scratch, (size_t)s->plan.resident_wgs * s->plan.wg_scratch_floats)))
    return bail(rc);
  s->workspace = ws;
  if (getenv("BNNHMC_DEBUG_PHASE")) {
    if ((rc = s->alloc(&s->debug_phase, (size_t)10 * 4096))) return bail(rc);
  }
  e = hipMemsetAsync(s->y, 0, (size_t)n_windows * s->n_pad * sizeof(float), s->stream);
  if (e == hipSuccess) e = hipMemsetAsync(ws, 0, s->workspace_bytes, s->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(s->stream);
  if (e != hipSuccess) {
    fail(BNNHMC_ERR_HIP, "clearing device memory failed: %s", hipGetErrorString(e));
    return bail(BNNHMC_ERR_HIP);
  }
  *out = s;
  return BNNHMC_OK;
}

int bnnhmc_destroy(bnnhmc_sampler* s) {
  if (!s) return BNNHMC_OK;
  if (s->stream) (void)hipStreamSynchronize(s->stream);
  for (void* p : s->allocs) (void)hipFree(p);
  if (s->ev0) (void)hipEventDestroy(s->ev0);
  if (s->ev1) (void)hipEventDestroy(s->ev1);
  if (s->ev_t0) (void)hipEventDestroy(s->ev_t0);
  if (s->ev_t1) (void)hipEventDestroy(s->ev_t1);
  if (s->stream) (void)hipStreamDestroy(s->stream);
  delete s;
  return BNNHMC_OK;
}

int bnnhmc_set_window_data(bnnhmc_sampler* s, int window, const float* x, const float* y) {
  if (!s || !x || !y) return fail(BNNHMC_ERR_INVALID, "null argument to bnnhmc_set_window_data");
  if (window < 0 || window >= s->n_windows)
    return fail(BNNHMC_ERR_INVALID, "window %d out of range [0, %d)", window, s->n_windows);
  const size_t nx = (size_t)s->model.n * s->model.d0;
  HIP_TRY(hipMemcpyAsync(s->X + (size_t)window * nx, x, nx * sizeof(float), hipMemcpyHostToDevice,
                         s->stream));
  HIP_TRY(hipMemcpyAsync(s->y + (size_t)window * s->n_pad, y, (size_t)s->model.n * sizeof(float),
                         hipMemcpyHostToDevice, s->stream));
  HIP_TRY(hipStreamSynchronize(s->stream));
  s->window_set[window] = 1;
  return BNNHMC_OK;
}

int bnnhmc_generate_window(bnnhmc_sampler* s, int window, float teacher_scale, float noise_sigma,
                           float* teacher_out) {
  if (!s) return fail(BNNHMC_ERR_INVALID, "sampler is null");
  if (window < 0 || window >= s->n_windows)
    return fail(BNNHMC_ERR_INVALID, "window %d out of range [0, %d)", window, s->n_windows);
  std::vector<float> X((size_t)s->model.n * s->model.d0), y(s->model.n);
  generate_window_host(s->hmc.seed, (uint32_t)window, s->model.n, s->model.d0, s->model.d1,
                       teacher_scale, noise_sigma, X.data(), y.data(), teacher_out);
  return bnnhmc_set_window_data(s, window, X.data(), y.data());
}

int bnnhmc_get_window_data(bnnhmc_sampler* s, int window, float* x_out, float* y_out) {
  if (!s) return fail(BNNHMC_ERR_INVALID, "sampler is null");
  if (window < 0 || window >= s->n_windows)
    return fail(BNNHMC_ERR_INVALID, "window %d out of range [0, %d)", window, s->n_windows);
  const size_t nx = (size_t)s->model.n * s->model.d0;
  if (x_out)
    HIP_TRY(hipMemcpyAsync(x_out, s->X + (size_t)window * nx, nx * sizeof(float),
                           hipMemcpyDeviceToHost, s->stream));
  if (y_out)
    HIP_TRY(hipMemcpyAsync(y_out, s->y + (size_t)window * s->n_pad,
                           (size_t)s->model.n * sizeof(float), hipMemcpyDeviceToHost, s->stream));
  HIP_TRY(hipStreamSynchronize(s->stream));
  return BNNHMC_OK;
}

int bnnhmc_init_chains(bnnhmc_sampler* s, const float* w0) {
  if (!s) return fail(BNNHMC_ERR_INVALID, "sampler is null");
  for (int w = 0; w < s->n_windows; ++w)
    if (!s->window_set[w])
      return fail(BNNHMC_ERR_STATE, "window %d has no data (set_window_data / generate_window)", w);
  const size_t C = s->n_chains;
  std::vector<float> hw(C * s->st_stride, 0.0f);
  if (w0)
    for (size_t c = 0; c < C; ++c) memcpy(&hw[c * s->st_stride], w0, sizeof(float) * s->L.P);
  HIP_TRY(hipMemcpyAsync(s->st_w, hw.data(), hw.size() * sizeof(float), hipMemcpyHostToDevice,
                         s->stream));
  HIP_TRY(launch_fill_f32(s->st_eps, C, s->hmc.eps0, s->stream));
  HIP_TRY(launch_fill_u32((unsigned*)s->st_t, C, 0u, s->stream));
  HIP_TRY(launch_fill_u32((unsigned*)s->st_sel, C, 0u, s->stream));
  HIP_TRY(launch_fill_u32((unsigned*)s->st_nacc, C, 0u, s->stream));
  // bootstrap (main.h:191-202): log-posterior rows and gradient at the initial state
  // (in the batches the transitions run in when all chains fit at once: a chain's sums are then added
  // in one order for its whole life)
  for (int base = 0, groups = 0; base < s->n_chains; base += groups) {
    groups = batch_size(s->plan, s->n_chains - base, s->batch_limit);
    KArgs a = base_args(s);
    a.mode = MODE_STEPS;
    a.L = 1;
    a.eps_in = 0.0f;
    a.chain_base = base;
    a.w_in = s->st_w + (size_t)base * s->st_stride;
    a.in_stride = s->st_stride;
    a.g_out = s->st_g + (size_t)base * s->st_stride;
    a.out_stride = s->st_stride;
    a.ell_out = s->ell0 + (size_t)base * s->n_pad;
    a.ell_stride = s->n_pad;
    int rc = launch_and_count(s, a, groups);
    if (rc) return rc;
  }
  int rc = check_status(s);
  if (rc) return rc;
  s->inited = true;
  s->transitions_done = 0;
  s->kernel_ms = 0.0;
  s->launches = 0;
  s->grad_evals = 0;
  return BNNHMC_OK;
}

int bnnhmc_run(bnnhmc_sampler* s, int n_transitions) {
  if (!s) return fail(BNNHMC_ERR_INVALID, "sampler is null");
  if (!s->inited) return fail(BNNHMC_ERR_STATE, "bnnhmc_init_chains has not been called");
  if (n_transitions < 0) return fail(BNNHMC_ERR_INVALID, "n_transitions must be >= 0");
  if (n_transitions == 0) return BNNHMC_OK;
  long launches = 0;
  HIP_TRY(hipEventRecord(s->ev0, s->stream));
  auto launch = [&](int base, int groups, int n_trans) -> int {
    KArgs a = base_args(s);
    a.mode = MODE_TRANSITIONS;
    a.n_trans = n_trans;
    a.chain_base = base;
    a.chain_wrap = s->n_chains;
    a.st_w = s->st_w;
    a.st_g = s->st_g;
    a.st_stride = s->st_stride;
    a.st_eps = s->st_eps;
    a.st_t = s->st_t;
    a.st_sel = s->st_sel;
    a.st_nacc = s->st_nacc;
    a.ell0 = s->ell0;
    a.ell1 = s->ell1;
    a.ell_stride = s->n_pad;
    a.samples = s->samples;
    a.n_samples = s->hmc.n_samples;
    a.burn_in = s->hmc.burn_in;
    a.adapt_steps = s->hmc.adapt_steps;
    a.dec_adj = -s->hmc.decrement / (1.0f + s->hmc.decrement);
    a.inc_adj = s->hmc.increment;
    a.log_target = (float)std::log((double)s->hmc.target_rate);
    a.tr_log_acpt = s->tr_la;
    a.tr_accept = s->tr_acc;
    a.tr_eps = s->tr_eps;
    a.trace_len = s->trace_len;
    a.seed = s->hmc.seed;
    a.rng_id_base = s->hmc.chain_id_base;
    a.debug_phase = s->debug_phase;
    const int rc = launch_and_count(s, a, groups);
    if (rc == BNNHMC_OK) ++launches;
    return rc;
  };
  // every chain of [base, base + count) (indices wrap at n_chains) runs n_trans transitions, in the
  // largest batches that fit
  auto run_range = [&](int base, int count, int n_trans) -> int {
    for (int groups = 0; count > 0; count -= groups, base = (base + groups) % s->n_chains) {
      groups = batch_size(s->plan, count, s->batch_limit);
      const int rc = launch(base, groups, n_trans);
      if (rc) return rc;
    }
    return BNNHMC_OK;
  };
  const int tpl = s->plan.transitions_per_launch;
  int full_batch = batch_size(s->plan, s->n_chains, s->batch_limit);
  int rc0 = BNNHMC_OK;
  if (s->plan.widen && !s->plan.wide && s->n_chains > full_batch) {
    // More chains than fit at once: they take turns.  A chain's run is cut into quanta of tpl transitions;
    // the quanta of all chains, in the order (pass, chain), are dealt to launches of full_batch chains
    // each, so that every launch but the last few fills the device with its widest batch (a fixed split
    // into batches would leave the last, small batch to run alone on wide, less efficient groups for the
    // whole call).  A launch never holds two quanta of one chain (full_batch < n_chains), and a chain's
    // quanta run in launch order.  What is left -- fewer than full_batch quanta, then the n mod tpl
    // transitions every chain still owes -- runs in the largest batches that fit.
    const long quanta = (long)s->n_chains * (n_transitions / tpl);
    long dealt = 0;
    // Which of the two batch shapes is faster depends on the card and on the data (see
    // resident_row_budget): the first launches of a call that is long enough are one of each, timed, and the
    // call (and the sampler, until a later call measures again) goes on with the faster.  Both do their
    // share of the work; from here on the results depend on a time measurement -- a run that must be
    // repeatable bit for bit sets cus_per_chain.
    const int wide_batch = batch_size(s->plan, s->n_chains);
    const int narrow_batch = s->batch_cap > 0 ? batch_size(s->plan, s->n_chains, s->batch_cap) : wide_batch;
    // (again only after kRetuneQuanta more quanta: a trial of the slower shape costs a few per cent of one
    // launch, and what is faster changes slowly, as the chains burn in)
    const long kRetuneQuanta = 2000;
    const bool due = s->quanta_since_tune < 0 || s->quanta_since_tune >= kRetuneQuanta;
    if (narrow_batch < wide_batch && env_batch_tune() && due && quanta >= narrow_batch + wide_batch) {
      const int trial[2] = {narrow_batch, wide_batch};
      for (int k = 0; k < 2 && rc0 == BNNHMC_OK; ++k) {
        HIP_TRY(hipEventRecord(s->ev_t0, s->stream));
        rc0 = launch((int)(dealt % s->n_chains), trial[k], tpl);
        HIP_TRY(hipEventRecord(s->ev_t1, s->stream));
        HIP_TRY(hipEventSynchronize(s->ev_t1));
        float tms = 0.0f;
        HIP_TRY(hipEventElapsedTime(&tms, s->ev_t0, s->ev_t1));
        s->tuned_rate[k] = tms > 0.0f ? (double)trial[k] * tpl * s->hmc.leapfrog_steps / tms : 0.0;
        dealt += trial[k];
      }
      if (rc0 == BNNHMC_OK) {
        s->batch_limit = s->tuned_rate[1] > s->tuned_rate[0] ? 0 : s->batch_cap;
        full_batch = batch_size(s->plan, s->n_chains, s->batch_limit);
        s->quanta_since_tune = quanta - dealt;
      }
    } else if (s->quanta_since_tune >= 0) {
      s->quanta_since_tune += quanta;
    }
    for (; rc0 == BNNHMC_OK && quanta - dealt >= full_batch; dealt += full_batch)
      rc0 = launch((int)(dealt % s->n_chains), full_batch, tpl);
    if (rc0 == BNNHMC_OK && quanta > dealt)
      rc0 = run_range((int)(dealt % s->n_chains), (int)(quanta - dealt), tpl);
    if (rc0 == BNNHMC_OK && n_transitions % tpl) rc0 = run_range(0, s->n_chains, n_transitions % tpl);
  } else {
    for (int base = 0, groups = 0; rc0 == BNNHMC_OK && base < s->n_chains; base += groups) {
      groups = batch_size(s->plan, s->n_chains - base, s->batch_limit);
      for (int done = 0; rc0 == BNNHMC_OK && done < n_transitions; done += tpl)
        rc0 = launch(base, groups, std::min(tpl, n_transitions - done));
    }
  }
  if (rc0) return rc0;
  HIP_TRY(hipEventRecord(s->ev1, s->stream));
  int rc = check_status(s);
  if (rc) return rc;
  float ms = 0.0f;
  HIP_TRY(hipEventElapsedTime(&ms, s->ev0, s->ev1));
  if (s->debug_phase) {
    // cycles per phase of the last launch, averaged over its workgroups
    std::vector<unsigned long long> h((size_t)10 * s->last_workgroups);
    HIP_TRY(hipMemcpy(h.data(), s->debug_phase, h.size() * sizeof(h[0]), hipMemcpyDeviceToHost));
    double tot[8] = {0};
    for (int wgi = 0; wgi < s->last_workgroups; ++wgi)
      for (int k = 0; k < 8; ++k) tot[k] += (double)h[(size_t)wgi * 10 + k] / s->last_workgroups;
    const char* names[8] = {"update+sync", "operand fetch", "tile loop", "partials->LDS+sync",
                            "stage1+store", "group barrier", "stage2", "epilogue"};
    double sum = 0;
    for (int k = 0; k < 8; ++k) sum += tot[k];
    for (int k = 0; k < 8; ++k)
      fprintf(stderr, "[bnnhmc phase] %-20s %14.0f ticks %6.2f%%\n", names[k], tot[k], 100.0 * tot[k] / sum);
    if (h[9] > 0)
      fprintf(stderr, "[bnnhmc phase] shader clock during the launch: %.0f MHz (%llu ticks in %.3f ms)\n",
              100.0 * (double)h[8] / (double)h[9], h[8], (double)h[9] * 1e-5);
  }
  s->kernel_ms += ms;
  s->launches += launches;
  s->grad_evals += (long)s->n_chains * n_transitions * s->hmc.leapfrog_steps;
  s->transitions_done += n_transitions;
  return BNNHMC_OK;
}

int bnnhmc_get_samples(bnnhmc_sampler* s, int chain, float* samples_out, int* n_stored) {
  if (!s) return fail(BNNHMC_ERR_INVALID, "sampler is null");
  if (chain < 0 || chain >= s->n_chains)
    return fail(BNNHMC_ERR_INVALID, "chain %d out of range [0, %d)", chain, s->n_chains);
  const int stored =
      std::max(0, std::min(s->hmc.n_samples, s->transitions_done - s->hmc.burn_in));
  if (n_stored) *n_stored = stored;
  if (samples_out && stored > 0) {
    HIP_TRY(hipMemcpyAsync(samples_out, s->samples + (size_t)chain * s->hmc.n_samples * s->L.P,
                           (size_t)stored * s->L.P * sizeof(float), hipMemcpyDeviceToHost,
                           s->stream));
    HIP_TRY(hipStreamSynchronize(s->stream));
  }
  return BNNHMC_OK;
}

int bnnhmc_get_chain_state(bnnhmc_sampler* s, int chain, float* w, float* grad, float* eps,
                           int* transitions_done, int* n_accepted) {
  if (!s) return fail(BNNHMC_ERR_INVALID, "sampler is null");
  if (chain < 0 || chain >= s->n_chains)
    return fail(BNNHMC_ERR_INVALID, "chain %d out of range [0, %d)", chain, s->n_chains);
  const size_t o = (size_t)chain * s->st_stride;
  if (w) HIP_TRY(hipMemcpyAsync(w, s->st_w + o, s->L.P * sizeof(float), hipMemcpyDeviceToHost, s->stream));
  if (grad)
    HIP_TRY(hipMemcpyAsync(grad, s->st_g + o, s->L.P * sizeof(float), hipMemcpyDeviceToHost, s->stream));
  if (eps) HIP_TRY(hipMemcpyAsync(eps, s->st_eps + chain, sizeof(float), hipMemcpyDeviceToHost, s->stream));
  if (transitions_done)
    HIP_TRY(hipMemcpyAsync(transitions_done, s->st_t + chain, sizeof(int), hipMemcpyDeviceToHost, s->stream));
  if (n_accepted)
    HIP_TRY(hipMemcpyAsync(n_accepted, s->st_nacc + chain, sizeof(int), hipMemcpyDeviceToHost, s->stream));
  HIP_TRY(hipStreamSynchronize(s->stream));
  return BNNHMC_OK;
}

int bnnhmc_set_chain_state(bnnhmc_sampler* s, int chain, const float* w, float eps,
                           int transitions_done, int n_accepted) {
  if (!s || !w) return fail(BNNHMC_ERR_INVALID, "null argument to bnnhmc_set_chain_state");
  if (chain < 0 || chain >= s->n_chains)
    return fail(BNNHMC_ERR_INVALID, "chain %d out of range [0, %d)", chain, s->n_chains);
  if (!s->inited) return fail(BNNHMC_ERR_STATE, "bnnhmc_init_chains has not been called");
  if (transitions_done < 0 || n_accepted < 0 || n_accepted > transitions_done)
    return fail(BNNHMC_ERR_INVALID, "bad transition counts");
  const size_t o = (size_t)chain * s->st_stride;
  const int zero = 0;
  HIP_TRY(hipMemcpyAsync(s->st_w + o, w, s->L.P * sizeof(float), hipMemcpyHostToDevice, s->stream));
  HIP_TRY(hipMemcpyAsync(s->st_eps + chain, &eps, sizeof(float), hipMemcpyHostToDevice, s->stream));
  HIP_TRY(hipMemcpyAsync(s->st_t + chain, &transitions_done, sizeof(int), hipMemcpyHostToDevice, s->stream));
  HIP_TRY(hipMemcpyAsync(s->st_nacc + chain, &n_accepted, sizeof(int), hipMemcpyHostToDevice, s->stream));
  HIP_TRY(hipMemcpyAsync(s->st_sel + chain, &zero, sizeof(int), hipMemcpyHostToDevice, s->stream));
  HIP_TRY(hipStreamSynchronize(s->stream));
  // gradient and per-row log-likelihood at w, exactly as the bootstrap step computes them
  KArgs a = base_args(s);
  a.mode = MODE_STEPS;
  a.L = 1;
  a.eps_in = 0.0f;
  a.chain_base = chain;
  a.w_in = s->st_w + o;
  a.in_stride = s->st_stride;
  a.g_out = s->st_g + o;
  a.out_stride = s->st_stride;
  a.ell_out = s->ell0 + (size_t)chain * s->n_pad;
  a.ell_stride = s->n_pad;
  int rc = launch_and_count(s, a, 1);
  if (rc) return rc;
  rc = check_status(s);
  if (rc) return rc;
  s->transitions_done = std::max(s->transitions_done, transitions_done);
  return BNNHMC_OK;
}

int bnnhmc_get_traces(bnnhmc_sampler* s, int chain, float* log_acpt, int* accepted, float* eps) {
  if (!s) return fail(BNNHMC_ERR_INVALID, "sampler is null");
  if (chain < 0 || chain >= s->n_chains)
    return fail(BNNHMC_ERR_INVALID, "chain %d out of range [0, %d)", chain, s->n_chains);
  const int len = std::min(s->transitions_done, s->trace_len);
  const size_t o = (size_t)chain * s->trace_len;
  if (len > 0) {
    if (log_acpt)
      HIP_TRY(hipMemcpyAsync(log_acpt, s->tr_la + o, len * sizeof(float), hipMemcpyDeviceToHost, s->stream));
    if (accepted)
      HIP_TRY(hipMemcpyAsync(accepted, s->tr_acc + o, len * sizeof(int), hipMemcpyDeviceToHost, s->stream));
    if (eps)
      HIP_TRY(hipMemcpyAsync(eps, s->tr_eps + o, len * sizeof(float), hipMemcpyDeviceToHost, s->stream));
    HIP_TRY(hipStreamSynchronize(s->stream));
  }
  return BNNHMC_OK;
}

int bnnhmc_eval(bnnhmc_sampler* s, int window, const float* w, float* ell, float* prior,
                float* grad) {
  if (!s || !w) return fail(BNNHMC_ERR_INVALID, "null argument to bnnhmc_eval");
  if (window < 0 || window >= s->n_windows)
    return fail(BNNHMC_ERR_INVALID, "window %d out of range [0, %d)", window, s->n_windows);
  if (!s->window_set[window]) return fail(BNNHMC_ERR_STATE, "window %d has no data", window);
  float* dw = s->tmp;
  float* dg = s->tmp + s->st_stride;
  float* dp = s->tmp + 2 * s->st_stride;
  HIP_TRY(hipMemcpyAsync(dw, w, s->L.P * sizeof(float), hipMemcpyHostToDevice, s->stream));
  int rc = eval_groups(s, window, dw, 0, 1, dg, dp, 0, s->tmp_ell, 0, nullptr);
  if (rc) return rc;
  rc = check_status(s);
  if (rc) return rc;
  if (ell)
    HIP_TRY(hipMemcpyAsync(ell, s->tmp_ell, (size_t)s->model.n * sizeof(float), hipMemcpyDeviceToHost, s->stream));
  if (prior)
    HIP_TRY(hipMemcpyAsync(prior, dp, s->L.P * sizeof(float), hipMemcpyDeviceToHost, s->stream));
  if (grad)
    HIP_TRY(hipMemcpyAsync(grad, dg, s->L.P * sizeof(float), hipMemcpyDeviceToHost, s->stream));
  HIP_TRY(hipStreamSynchronize(s->stream));
  return BNNHMC_OK;
}

int bnnhmc_final_loss(bnnhmc_sampler* s, int chain, double* loss1, double* loss2, double* full) {
  if (!s) return fail(BNNHMC_ERR_INVALID, "sampler is null");
  if (chain < 0 || chain >= s->n_chains)
    return fail(BNNHMC_ERR_INVALID, "chain %d out of range [0, %d)", chain, s->n_chains);
  const int stored =
      std::max(0, std::min(s->hmc.n_samples, s->transitions_done - s->hmc.burn_in));
  if (stored == 0) return fail(BNNHMC_ERR_STATE, "chain %d has no kept samples yet", chain);
  const int window = chain / s->cpw;
  const float* base = s->samples + (size_t)chain * s->hmc.n_samples * s->L.P;
  std::vector<double> sums((size_t)2 * s->plan.max_groups);
  double l1 = 0, l2 = 0, fl = 0;
  int step = 0;
  // the samples are evaluated max_groups at a time, one chain group per sample
  for (int b = 0; b < stored; b += s->plan.max_groups) {
    const int groups = std::min(s->plan.max_groups, stored - b);
    int rc = eval_groups(s, window, base + (size_t)b * s->L.P, s->L.P, groups, nullptr, nullptr, 0,
                         nullptr, 0, s->tmp_sums);
    if (rc) return rc;
    rc = check_status(s);
    if (rc) return rc;
    HIP_TRY(hipMemcpy(sums.data(), s->tmp_sums, (size_t)2 * groups * sizeof(double),
                      hipMemcpyDeviceToHost));
    for (int i = 0; i < groups; ++i, ++step) {
      // running means as main.h:106-111; the reference's per-sample sums are FP32
      const double s1 = (double)(float)sums[2 * i], s2 = (double)(float)sums[2 * i + 1];
      const double ds = (double)step;
      l1 = (l1 * ds + s1) / (ds + 1);
      l2 = (l2 * ds + s2) / (ds + 1);
      fl = (fl * ds + (s1 + s2)) / (ds + 1);
    }
  }
  if (loss1) *loss1 = l1;
  if (loss2) *loss2 = l2;
  if (full) *full = fl;
  return BNNHMC_OK;
}

int bnnhmc_split_rhat_ess(const float* samples, int n_chains, int n_samples, int n_params,
                          size_t chain_stride, double* rhat, double* ess) {
  if (!samples) return fail(BNNHMC_ERR_INVALID, "samples is null");
  if (n_chains < 1 || n_params < 1) return fail(BNNHMC_ERR_INVALID, "need at least one chain and one parameter");
  if (n_samples < 8) return fail(BNNHMC_ERR_INVALID, "need at least 8 draws per chain, got %d", n_samples);
  const int n = n_samples / 2, m = 2 * n_chains;
  std::vector<double> x((size_t)m * n), mean(m), var(m), acov_mean(n), rho(n);
  for (int p = 0; p < n_params; ++p) {
    // sequence 2c is the first half of chain c, 2c + 1 its last n draws
    for (int c = 0; c < n_chains; ++c)
      for (int h = 0; h < 2; ++h) {
        const int first = h == 0 ? 0 : n_samples - n;
        double* dst = x.data() + (size_t)(2 * c + h) * n;
        for (int i = 0; i < n; ++i)
          dst[i] = (double)samples[(size_t)c * chain_stride + (size_t)(first + i) * n_params + p];
      }
    double grand = 0.0, W = 0.0;
    for (int j = 0; j < m; ++j) {
      const double* xs = x.data() + (size_t)j * n;
      double s1 = 0.0;
      for (int i = 0; i < n; ++i) s1 += xs[i];
      mean[j] = s1 / n;
      double s2 = 0.0;
      for (int i = 0; i < n; ++i) s2 += (xs[i] - mean[j]) * (xs[i] - mean[j]);
      var[j] = s2 / (n - 1);
      grand += mean[j] / m;
      W += var[j] / m;
    }
    double B_over_n = 0.0;
    for (int j = 0; j < m; ++j) B_over_n += (mean[j] - grand) * (mean[j] - grand) / (m - 1);
    const double var_plus = (double)(n - 1) / n * W + B_over_n;
    if (!(W > 0.0)) {
      if (rhat) rhat[p] = 1.0;
      if (ess) ess[p] = (double)m * n;
      continue;
    }
    if (rhat) rhat[p] = std::sqrt(var_plus / W);
    if (!ess) continue;
    // rho_t for t = 0, 1, ... computed on demand; acov_j(t) with the 1 / (n - 1) normalisation
    auto rho_at = [&](int t) {
      double a = 0.0;
      for (int j = 0; j < m; ++j) {
        const double* xs = x.data() + (size_t)j * n;
        double s = 0.0;
        for (int i = 0; i + t < n; ++i) s += (xs[i] - mean[j]) * (xs[i + t] - mean[j]);
        a += s / (n - 1) / m;
      }
      return 1.0 - (W - a) / var_plus;
    };
    // Geyer's initial positive sequence of pair sums, made monotone non-increasing
    double tau = -1.0, prev_pair = 0.0;
    bool have_prev = false;
    for (int t = 0; t + 1 < n; t += 2) {
      double pair = rho_at(t) + rho_at(t + 1);
      if (!(pair > 0.0)) break;
      if (have_prev && pair > prev_pair) pair = prev_pair;
      tau += 2.0 * pair;
      prev_pair = pair;
      have_prev = true;
    }
    const double mn = (double)m * n;
    tau = std::max(tau, 1.0 / std::log10(mn));
    ess[p] = mn / tau;
  }
  return BNNHMC_OK;
}

int bnnhmc_window_diagnostics(bnnhmc_sampler* s, int window, double* rhat, double* ess) {
  if (!s) return fail(BNNHMC_ERR_INVALID, "sampler is null");
  if (window < 0 || window >= s->n_windows)
    return fail(BNNHMC_ERR_INVALID, "window %d out of range [0, %d)", window, s->n_windows);
  const int stored =
      std::max(0, std::min(s->hmc.n_samples, s->transitions_done - s->hmc.burn_in));
  if (stored < 8)
    return fail(BNNHMC_ERR_STATE, "window %d has %d kept samples per chain; 8 are needed", window, stored);
  const size_t stride = (size_t)s->hmc.n_samples * s->L.P;
  std::vector<float> host((size_t)s->cpw * stride);
  HIP_TRY(hipMemcpyAsync(host.data(), s->samples + (size_t)window * s->cpw * stride,
                         host.size() * sizeof(float), hipMemcpyDeviceToHost, s->stream));
  HIP_TRY(hipStreamSynchronize(s->stream));
  return bnnhmc_split_rhat_ess(host.data(), s->cpw, stored, s->L.P, stride, rhat, ess);
}

int bnnhmc_get_batching(bnnhmc_sampler* s, int* chains_per_launch, int* workgroups_per_chain,
                        double* trial_rates) {
  if (!s) return fail(BNNHMC_ERR_INVALID, "sampler is null");
  const int groups = batch_size(s->plan, s->n_chains, s->batch_limit);
  if (chains_per_launch) *chains_per_launch = groups;
  if (workgroups_per_chain)
    *workgroups_per_chain =
        s->plan.widen ? widen_group(s->plan.G, groups, s->plan.resident_wgs, 256) : s->plan.G;
  if (trial_rates) {
    trial_rates[0] = s->tuned_rate[0] * 1e3;
    trial_rates[1] = s->tuned_rate[1] * 1e3;
  }
  return BNNHMC_OK;
}

int bnnhmc_get_timing(bnnhmc_sampler* s, double* kernel_ms, long* launches, long* grad_evals,
                      int* workgroups) {
  if (!s) return fail(BNNHMC_ERR_INVALID, "sampler is null");
  if (kernel_ms) *kernel_ms = s->kernel_ms;
  if (launches) *launches = s->launches;
  if (grad_evals) *grad_evals = s->grad_evals;
  if (workgroups) *workgroups = s->last_workgroups;
  return BNNHMC_OK;
}

}  // extern "C"
