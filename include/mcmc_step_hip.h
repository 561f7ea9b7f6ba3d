/*
 * mcmc_step_hip.h -- the operator header of NVIDIA/mcmc-bnn-example for an MI355X (gfx950), on top of the
 * C ABI in bnn_hmc.h.
 *
 * A third branch beside include/mcmc/mcmc_step_ffma.h and include/mcmc/mcmc_step_tc.h (selected in
 * include/mcmc/main.h:38-42): it offers everything the reference's driver takes from its operator header --
 *   mcmc_step<T, LP_STEPS>(...)                    include/mcmc/mcmc_step_ffma.h:395-427, mcmc_step_tc.h:679-696
 *   set_dynamic_smem_max_size<T>()                 mcmc_step_ffma.h:429-436          (main.h:120)
 *   full_smem_size<T>(), leapfrog_max_smem_size<T>()   mcmc_step_ffma.h:57-70       (main.h:121-125)
 *   N_THREADS, N_WARPS, N_BLKS, N_WARP_SAMPLES, N_BLK_SAMPLES, N_P_ALIGNED   mcmc_step_ffma.h:46-52 (main.h:52-59, 121-123)
 * -- with the same names and argument meaning.  Differences a caller must know are listed at mcmc_step below.
 *
 * Expects, as the two reference headers do, that the including file has already brought in
 * global_params.h (FEAT_DIM, NUM_PARAMS, N_SAMPLES and the model constants), utils_matrix.h
 * (DeviceMatrix<T> with ptr() and nbytes(), utils_matrix.h:67-69) and an ASSERT(cond, fmt, ...) macro
 * (utils_cuda.h:30-46).  The stream type is hipStream_t (void* here, so that no HIP header is needed).
 */
#ifndef MCMC_STEP_HIP_H
#define MCMC_STEP_HIP_H

#include <cstddef>
#include <cstdio>
#include <cstdlib>

#include "bnn_hmc.h"

#ifndef ASSERT
#define ASSERT(cond, fmt, ...)                                                       \
  do {                                                                               \
    if (!(cond)) {                                                                   \
      std::fprintf(stderr, "Assertion failed at %s:%d: " fmt "\n", __FILE__, __LINE__, ##__VA_ARGS__); \
      std::abort();                                                                  \
    }                                                                                \
  } while (0)
#endif

/* the reference sets the rows per warp on the compiler's command line; here the library decides */
#ifdef N_WARP_SAMPLES
#undef N_WARP_SAMPLES
#endif

namespace mcmc {

/* One chain on the whole device: 256 workgroups (one per compute unit) of 512 threads = 8 wavefronts of
 * 64 lanes; the rows go to the wavefronts in runs of whole 16-row tiles. */
static constexpr int N_THREADS = 512;
static constexpr int N_WARPS = N_THREADS / 64;
static constexpr int N_BLKS = 256;
static constexpr int N_WARP_SAMPLES = 16 * (((N_SAMPLES + 15) / 16 + N_BLKS * N_WARPS - 1) / (N_BLKS * N_WARPS));
static constexpr int N_BLK_SAMPLES = N_WARP_SAMPLES * N_WARPS;
static constexpr int IVECLEN = 4;
static constexpr int N_P_ALIGNED = (NUM_PARAMS + IVECLEN - 1) / IVECLEN * IVECLEN;

/* The model of global_params.h:39-61 and the launch the constants above describe. */
inline const bnnhmc_model& hip_model() {
  static const bnnhmc_model m = [] {
    bnnhmc_model v;
    bnnhmc_default_model(&v); /* Student-t scale 100, 2.2 degrees of freedom, prior scale 200 */
    v.d0 = FEAT_DIM[0];
    v.d1 = FEAT_DIM[1];
    v.n = N_SAMPLES;
    return v;
  }();
  return m;
}
inline const bnnhmc_launch& hip_launch() {
  static const bnnhmc_launch l = [] {
    bnnhmc_launch v;
    bnnhmc_default_launch(&v);
    v.cus_per_chain = N_BLKS;
    v.threads = N_THREADS;
    return v;
  }();
  return l;
}

/* LDS bytes a workgroup of the trajectory kernel uses, and the most a workgroup may use on this device
 * (the driver prints both, main.h:121-125).  Asked of the library, which asks the device. */
template <typename T>
inline int full_smem_size() {
  size_t lds = 0;
  const int rc = bnnhmc_step_launch_info(&hip_model(), &hip_launch(), nullptr, nullptr, nullptr, &lds, nullptr);
  ASSERT(rc == BNNHMC_OK, "%s", bnnhmc_last_error());
  return (int)lds;
}
template <typename T>
inline int leapfrog_max_smem_size() {
  size_t lds_max = 0;
  const int rc = bnnhmc_step_launch_info(&hip_model(), &hip_launch(), nullptr, nullptr, nullptr, nullptr, &lds_max);
  ASSERT(rc == BNNHMC_OK, "%s", bnnhmc_last_error());
  return (int)lds_max;
}
/* Nothing for the caller to set: the library sets its kernels' attributes when it first plans a launch.
 * Planning it here keeps that work out of the first timed mcmc_step (main.h:120 comes before t_start). */
template <typename T>
inline void set_dynamic_smem_max_size() {
  int wgs = 0, threads = 0, rows = 0;
  const int rc = bnnhmc_step_launch_info(&hip_model(), &hip_launch(), &wgs, &threads, &rows, nullptr, nullptr);
  ASSERT(rc == BNNHMC_OK, "%s", bnnhmc_last_error());
  ASSERT(wgs == N_BLKS && threads == N_THREADS && rows == N_WARP_SAMPLES,
         "the library plans %d workgroups x %d threads, %d rows per wavefront; this header says %d x %d, %d", wgs,
         threads, rows, N_BLKS, N_THREADS, N_WARP_SAMPLES);
}

/* ints of the grid_sync_workspace this operator needs (main.h:169-173 allocates LEAPFROG_STEPS ints for
 * the tensor-core variant): DeviceMatrix<int> gsw(1, step_workspace_ints(), 0, stream); */
inline size_t step_workspace_ints() {
  return (bnnhmc_step_workspace_bytes(&hip_model(), &hip_launch()) + sizeof(int) - 1) / sizeof(int);
}

/*
 * LP_STEPS fused leapfrog steps in one launch.  Same arguments as the reference's operator.  Differences:
 *  - grid_sync_workspace must be given (step_workspace_ints() ints; it needs no initialisation);
 *  - results always land in the buffers NAMED weights_next, mom_next, grad_cur, loss_values, and grad_next
 *    is zeroed: the caller's views are not rotated as mcmc_step_ffma.h:414,421 does, and no
 *    (LP_STEPS - 1) % 3 replay of do_swap_g is owed as after mcmc_step_tc.h (main.h:224-227);
 *  - weights_prev, mom_prev, grad_prev are only read, so grad_cur need not be zero on entry;
 *  - a failure inside the kernel (bounded wait expired, workgroups disagree) is reported by
 *    bnnhmc_step_check(&hip_model(), &hip_launch(), grid_sync_workspace->ptr(), stream), which
 *    synchronises; one check after any number of steps is enough.
 */
template <typename T, int LP_STEPS = 1, typename Stream = void*>
void mcmc_step(const DeviceMatrix<T>& x, const DeviceMatrix<T>& y, DeviceMatrix<T>& weights_prev,
               DeviceMatrix<T>& weights_next, DeviceMatrix<T>& mom_prev, DeviceMatrix<T>& mom_next,
               DeviceMatrix<T>& grad_prev, DeviceMatrix<T>& grad_cur, DeviceMatrix<T>& grad_next,
               DeviceMatrix<T>& loss_values, DeviceMatrix<int>* grid_sync_workspace, T eps, const Stream& stream) {
  static_assert(sizeof(T) == sizeof(float), "the library computes in FP32");
  static_assert(LP_STEPS > 0, "LP_STEPS must be >0");
  ASSERT(grid_sync_workspace != nullptr, "Expecting a grid sync workspace of %zu ints", step_workspace_ints());
  const int rc = bnnhmc_mcmc_step(&hip_model(), &hip_launch(), x.ptr(), y.ptr(), weights_prev.ptr(),
                                  weights_next.ptr(), mom_prev.ptr(), mom_next.ptr(), grad_prev.ptr(), grad_cur.ptr(),
                                  grad_next.ptr(), loss_values.ptr(), grid_sync_workspace->ptr(),
                                  grid_sync_workspace->nbytes(), eps, LP_STEPS, (void*)stream);
  ASSERT(rc == BNNHMC_OK, "%s", bnnhmc_last_error());
}

}  // namespace mcmc
#endif
