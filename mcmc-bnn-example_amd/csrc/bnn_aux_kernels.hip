// Small kernels around the trajectory kernel: fills, momentum sampling, the log-accept reduction and
// the loss sums of the operator-level entry points.
#include <hip/hip_runtime.h>

#include "bnn_kernels.h"
#include "bnn_rng.h"

namespace bnn {

__global__ void fill_u32_kernel(unsigned* p, size_t n, unsigned v) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x)
    p[i] = v;
}
__global__ void fill_f32_kernel(float* p, size_t n, float v) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x)
    p[i] = v;
}

static int fill_blocks(size_t n) {
  size_t b = (n + 255) / 256;
  return (int)(b < 1 ? 1 : (b > 2048 ? 2048 : b));
}
hipError_t launch_fill_u32(unsigned* p, size_t n, unsigned v, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(fill_u32_kernel, dim3(fill_blocks(n)), dim3(256), 0, stream, p, n, v);
  return hipGetLastError();
}
hipError_t launch_fill_f32(float* p, size_t n, float v, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(fill_f32_kernel, dim3(fill_blocks(n)), dim3(256), 0, stream, p, n, v);
  return hipGetLastError();
}

// Status words of a step-operator workspace: cleared only when the workspace has not been used before
// (it then holds whatever the caller's allocation held), which the last two status words tell: the
// library leaves a 64-bit mark there once it has cleared the others.  A record of a failed step thus
// stays until bnnhmc_step_check has reported it, however many steps were queued behind it.
constexpr unsigned STATUS_MARK0 = 0x626e6e68u, STATUS_MARK1 = 0x6d637374u;
__global__ void prepare_status_kernel(unsigned* status) {
  const unsigned m0 = status[STATUS_WORDS - 2], m1 = status[STATUS_WORDS - 1];
  __syncthreads();
  if (m0 == STATUS_MARK0 && m1 == STATUS_MARK1) return;
  const int t = (int)threadIdx.x;
  if (t < STATUS_WORDS - 2) status[t] = 0u;
  else if (t == STATUS_WORDS - 2) status[t] = STATUS_MARK0;
  else if (t == STATUS_WORDS - 1) status[t] = STATUS_MARK1;
}
hipError_t launch_prepare_status(unsigned* status, hipStream_t stream) {
  static_assert(STATUS_WORDS == 64, "one thread per status word");
  hipLaunchKernelGGL(prepare_status_kernel, dim3(1), dim3(STATUS_WORDS), 0, stream, status);
  return hipGetLastError();
}
// clears a reported record, leaving the mark in place
hipError_t launch_clear_status(unsigned* status, hipStream_t stream) {
  return launch_fill_u32(status, STATUS_WORDS - 2, 0u, stream);
}

// Runs after every launch of a trajectory kernel: all workgroups of a chain group must report the
// same state hash.  The first mismatch is recorded in the status words ([4] workgroup index + 1,
// [5] its chain group, [6..9] the two hashes); a launch that was abandoned (status[0] set) left no
// hashes to compare.
__global__ void compare_hashes_kernel(const unsigned long long* h, int wgs, int G, unsigned* status) {
  if (status[0] != 0u) return;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < wgs; i += gridDim.x * blockDim.x) {
    const int lead = i / G * G;
    if (h[i] != h[lead] && atomicCAS(status + 4, 0u, (unsigned)i + 1u) == 0u) {
      status[5] = (unsigned)(i / G);
      status[6] = (unsigned)h[i];
      status[7] = (unsigned)(h[i] >> 32);
      status[8] = (unsigned)h[lead];
      status[9] = (unsigned)(h[lead] >> 32);
    }
  }
}
hipError_t launch_compare_hashes(const unsigned long long* h, int wgs, int G, unsigned* status,
                                 hipStream_t stream) {
  hipLaunchKernelGGL(compare_hashes_kernel, dim3(1), dim3(256), 0, stream, h, wgs, G, status);
  return hipGetLastError();
}

// main.h:207-216 with the counter-based generator
__global__ void sample_momentum_kernel(uint32_t seed, uint32_t chain_id, uint32_t transition, int n,
                                       float* a, float* b) {
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
    const float v = rng_normal(seed, chain_id, STREAM_MOMENTUM, transition, (uint64_t)i);
    if (a) a[i] = v;
    if (b) b[i] = v;
  }
}
hipError_t launch_sample_momentum(uint32_t seed, uint32_t chain_id, uint32_t transition, int n,
                                  float* a, float* b, hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  hipLaunchKernelGGL(sample_momentum_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, seed,
                     chain_id, transition, n, a, b);
  return hipGetLastError();
}

// deterministic sum of per-thread doubles over one 1024-thread workgroup; result in every thread
__device__ double block_sum_1024(double v, double* s_buf) {
  for (int msk = 1; msk < 64; msk <<= 1) {
    const uint64_t b = double_to_bits(v);
    const uint32_t lo = (uint32_t)__shfl_xor((int)(uint32_t)b, msk);
    const uint32_t hi = (uint32_t)__shfl_xor((int)(uint32_t)(b >> 32), msk);
    v += bits_to_double(((uint64_t)hi << 32) | lo);
  }
  __syncthreads();
  if ((threadIdx.x & 63) == 0) s_buf[threadIdx.x >> 6] = v;
  __syncthreads();
  double tot = 0.0;
  for (int w = 0; w < (int)(blockDim.x >> 6); ++w) tot += s_buf[w];
  return tot;
}

// kernel_helpers.h:163-175: per-element FP32 terms, summed in double in a fixed order
__global__ __launch_bounds__(1024) void log_acpt_kernel(int n_loss, int n_mom, const float* prev_loss,
                                                        const float* new_loss, const float* prev_mom,
                                                        const float* new_mom, const float* grad_cur,
                                                        float eps, float* out) {
  __shared__ double s_buf[16];
  double acc = 0.0;
  for (int i = threadIdx.x; i < n_loss; i += blockDim.x) acc += (double)(new_loss[i] - prev_loss[i]);
  for (int i = threadIdx.x; i < n_mom; i += blockDim.x) {
    const float nm = __builtin_fmaf(eps * 0.5f, grad_cur[i], new_mom[i]);
    float t = prev_mom[i] * prev_mom[i];
    t = __builtin_fmaf(-nm, nm, t);
    acc += (double)(0.5f * t);
  }
  const double tot = block_sum_1024(acc, s_buf);
  if (threadIdx.x == 0) out[0] = (float)tot;
}
hipError_t launch_log_acpt(int n_loss, int n_mom, const float* prev_loss, const float* new_loss,
                           const float* prev_mom, const float* new_mom, const float* grad_cur,
                           float eps, float* out, hipStream_t stream) {
  hipLaunchKernelGGL(log_acpt_kernel, dim3(1), dim3(1024), 0, stream, n_loss, n_mom, prev_loss,
                     new_loss, prev_mom, new_mom, grad_cur, eps, out);
  return hipGetLastError();
}

// kernel_helpers.h:205-210: sum of the first n entries and of the next n_params entries
__global__ __launch_bounds__(1024) void loss_sums_kernel(const float* lv, int n, int n_params,
                                                         float* out2) {
  __shared__ double s_buf[16];
  double a = 0.0, b = 0.0;
  for (int i = threadIdx.x; i < n; i += blockDim.x) a += (double)lv[i];
  for (int i = threadIdx.x; i < n_params; i += blockDim.x) b += (double)lv[n + i];
  const double ta = block_sum_1024(a, s_buf);
  const double tb = block_sum_1024(b, s_buf);
  if (threadIdx.x == 0) {
    out2[0] = (float)ta;
    out2[1] = (float)tb;
  }
}
hipError_t launch_loss_sums(const float* loss_values, int n, int n_params, float* out2,
                            hipStream_t stream) {
  hipLaunchKernelGGL(loss_sums_kernel, dim3(1), dim3(1024), 0, stream, loss_values, n, n_params,
                     out2);
  return hipGetLastError();
}

}  // namespace bnn
