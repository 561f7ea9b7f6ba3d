// Compiles include/mcmc_step_hip.h the way the reference's driver would use it -- against stand-ins for
// the few things that header expects from the reference's own headers (the constants of
// include/mcmc/global_params.h and a DeviceMatrix<T> with ptr() / nbytes(), include/mcmc/utils_matrix.h:
// 67-69) -- and walks the start of mcmc::main_loop (include/mcmc/main.h:117-232) through it: the launch
// banner, the bootstrap step, momentum resampling, the buffer rotation, one trajectory, the log accept
// ratio and the loss sums.  Plain C++ (g++), linked against libbnn_hmc.so and the HIP runtime.
//
//   shim_check [seed]      prints one line per quantity; exit status 3 when no GPU is visible
#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <utility>
#include <vector>

// ---- stand-in for include/mcmc/global_params.h (same names; a short trajectory) ----
namespace mcmc {
static constexpr int LEAPFROG_STEPS = 40;
static constexpr int FEAT_DIM[] = {22, 40, 1};
static constexpr int NUM_LAYERS = 2;
static constexpr int NUM_PARAMS = FEAT_DIM[0] * FEAT_DIM[1] + FEAT_DIM[1] + FEAT_DIM[1] * FEAT_DIM[2] + FEAT_DIM[2];
static constexpr int N_SAMPLES = 58368;
static constexpr int N_COLS = FEAT_DIM[0];
static constexpr unsigned SEED_INIT = 1;
static constexpr double STEP_SIZE_INIT = 0.01;

#define HIP_OK(call)                                                                        \
  do {                                                                                      \
    hipError_t e_ = (call);                                                                 \
    if (e_ != hipSuccess) {                                                                 \
      std::fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));                \
      std::exit(1);                                                                         \
    }                                                                                       \
  } while (0)

// ---- stand-in for DeviceMatrix<T> (utils_matrix.h): owning or a view, ptr(), nbytes(), swap() ----
template <typename T>
class DeviceMatrix {
  bool view;
  size_t M, N;
  T* data;

 public:
  DeviceMatrix(size_t m, size_t n) : view(false), M(m), N(n), data(nullptr) { HIP_OK(hipMalloc((void**)&data, nbytes())); }
  DeviceMatrix(size_t m, size_t n, T init, hipStream_t st) : DeviceMatrix(m, n) {
    std::vector<T> h(m * n, init);
    HIP_OK(hipMemcpyAsync(data, h.data(), nbytes(), hipMemcpyHostToDevice, st));
    HIP_OK(hipStreamSynchronize(st));
  }
  DeviceMatrix(size_t m, size_t n, T* p) : view(true), M(m), N(n), data(p) {}
  DeviceMatrix(const DeviceMatrix&) = delete;
  ~DeviceMatrix() {
    if (!view) (void)hipFree(data);
  }
  const T* ptr() const { return data; }
  T* ptr() { return data; }
  size_t nel() const { return M * N; }
  size_t nbytes() const { return nel() * sizeof(T); }
  void swap(DeviceMatrix& o) noexcept {
    std::swap(view, o.view);
    std::swap(M, o.M);
    std::swap(N, o.N);
    std::swap(data, o.data);
  }
};
}  // namespace mcmc

#include "mcmc_step_hip.h"

namespace mcmc {
// main.h:48-76
template <typename T>
struct Network {
  Network(hipStream_t st)
      : block(7, N_P_ALIGNED, T(0), st),
        w_prev(1, N_P_ALIGNED, block.ptr()),
        w_next(1, N_P_ALIGNED, block.ptr() + N_P_ALIGNED * 3),
        mom_prev(1, N_P_ALIGNED, block.ptr() + N_P_ALIGNED * 1),
        mom_next(1, N_P_ALIGNED, block.ptr() + N_P_ALIGNED * 6),
        grad_prev(1, N_P_ALIGNED, block.ptr() + N_P_ALIGNED * 2),
        grad_cur(1, N_P_ALIGNED, block.ptr() + N_P_ALIGNED * 4),
        grad_next(1, N_P_ALIGNED, block.ptr() + N_P_ALIGNED * 5) {}
  DeviceMatrix<T> block;
  DeviceMatrix<T> w_prev, w_next, mom_prev, mom_next, grad_prev, grad_cur, grad_next;
  void do_swap_g() {
    grad_cur.swap(grad_next);
    grad_prev.swap(grad_next);
  }
  void do_swap() {
    w_prev.swap(w_next);
    mom_prev.swap(mom_next);
    do_swap_g();
  }
};

template <typename T>
int main_loop_start(unsigned seed) {
  // main.h:120-125
  set_dynamic_smem_max_size<T>();
  std::cout << "Using " << N_WARP_SAMPLES << " rows/warp -> " << N_BLKS << " blocks with " << N_BLK_SAMPLES
            << " rows / block. Using " << leapfrog_max_smem_size<T>() << " max shared mem size (fit the required "
            << full_smem_size<T>() << " smem)." << std::endl;
  hipStream_t stream = nullptr;
  // main.h:156-159: the data set (here the synthetic recipe of window 0 instead of read_data)
  DeviceMatrix<T> data(N_SAMPLES, N_COLS);
  DeviceMatrix<T> labels(N_SAMPLES, FEAT_DIM[NUM_LAYERS]);
  {
    std::vector<float> x((size_t)N_SAMPLES * N_COLS), y(N_SAMPLES);
    if (bnnhmc_generate_window_host(seed, 0, N_SAMPLES, FEAT_DIM[0], FEAT_DIM[1], 0.3f, 5.0f, x.data(), y.data(),
                                    nullptr) != BNNHMC_OK)
      return 1;
    HIP_OK(hipMemcpy(data.ptr(), x.data(), data.nbytes(), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(labels.ptr(), y.data(), labels.nbytes(), hipMemcpyHostToDevice));
  }
  // main.h:166-183
  Network<T> net(stream);
  DeviceMatrix<T> loss_values(1, N_SAMPLES + NUM_PARAMS);
  DeviceMatrix<T> loss_red_values(1, 3);
  DeviceMatrix<int> gsw(1, step_workspace_ints());  // the grid_sync_workspace of this operator
  DeviceMatrix<int>* grid_sync_workspace = &gsw;
  DeviceMatrix<T> prev_step_loss(1, N_SAMPLES + NUM_PARAMS);
  DeviceMatrix<T> prev_lp_mom(1, NUM_PARAMS);
  // main.h:191-202: bootstrap
  T eps = (T)STEP_SIZE_INIT;
  mcmc_step<T, 1>(data, labels, net.w_prev, net.w_next, net.mom_prev, net.mom_next, net.grad_prev, net.grad_cur,
                  net.grad_next, loss_values, grid_sync_workspace, eps, stream);
  HIP_OK(hipMemcpyAsync(prev_step_loss.ptr(), loss_values.ptr(), loss_values.nbytes(), hipMemcpyDeviceToDevice,
                        stream));
  float l1 = 0, l2 = 0;
  if (bnnhmc_get_loss_values(loss_values.ptr(), N_SAMPLES, NUM_PARAMS, &l1, &l2, stream) != BNNHMC_OK) return 1;
  std::printf("bootstrap loss1 %.9g loss2 %.9g\n", l1, l2);
  // main.h:204-218: momentum of transition 0 (counter-based generator instead of the thrust lambda)
  if (bnnhmc_sample_momentum(SEED_INIT, 0, 0, NUM_PARAMS, prev_lp_mom.ptr(), net.mom_next.ptr(), stream) != BNNHMC_OK)
    return 1;
  net.do_swap();
  // main.h:220-223: the trajectory.  The results are in the buffers named *_next / grad_cur: no replay of
  // do_swap_g (main.h:224-227) with this operator
  mcmc_step<T, LEAPFROG_STEPS>(data, labels, net.w_prev, net.w_next, net.mom_prev, net.mom_next, net.grad_prev,
                               net.grad_cur, net.grad_next, loss_values, grid_sync_workspace, eps, stream);
  // main.h:228-232: the log accept ratio
  float h_log_acpt = 0;
  if (bnnhmc_log_acpt(N_SAMPLES + NUM_PARAMS, NUM_PARAMS, prev_step_loss.ptr(), loss_values.ptr(), prev_lp_mom.ptr(),
                      net.mom_next.ptr(), net.grad_cur.ptr(), eps, loss_red_values.ptr() + 2, &h_log_acpt,
                      stream) != BNNHMC_OK)
    return 1;
  const int rc = bnnhmc_step_check(&hip_model(), &hip_launch(), gsw.ptr(), stream);
  if (rc != BNNHMC_OK) {
    std::fprintf(stderr, "step check: %s\n", bnnhmc_last_error());
    return 1;
  }
  if (bnnhmc_get_loss_values(loss_values.ptr(), N_SAMPLES, NUM_PARAMS, &l1, &l2, stream) != BNNHMC_OK) return 1;
  std::vector<float> w(NUM_PARAMS), g(NUM_PARAMS);
  HIP_OK(hipMemcpy(w.data(), net.w_next.ptr(), NUM_PARAMS * sizeof(float), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(g.data(), net.grad_cur.ptr(), NUM_PARAMS * sizeof(float), hipMemcpyDeviceToHost));
  std::printf("steps %d eps %.9g\n", LEAPFROG_STEPS, (double)eps);
  std::printf("log_acpt %.9g\n", h_log_acpt);
  std::printf("proposal loss1 %.9g loss2 %.9g\n", l1, l2);
  std::printf("w_next");
  for (int p = 0; p < NUM_PARAMS; p += 120) std::printf(" %.9g", w[p]);
  std::printf("\ngrad_cur");
  for (int p = 0; p < NUM_PARAMS; p += 120) std::printf(" %.9g", g[p]);
  std::printf("\n");
  return 0;
}
}  // namespace mcmc

int main(int argc, char** argv) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
    std::fprintf(stderr, "no HIP device visible\n");
    return 3;
  }
  return mcmc::main_loop_start<float>(argc > 1 ? (unsigned)std::strtoul(argv[1], nullptr, 10) : 0u);
}
