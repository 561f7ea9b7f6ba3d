// Host-callable launchers of the library's kernels (implemented in the .hip files).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "bnn_device.h"

namespace bnn {

// trajectory kernel for (d0, d1, layer, likelihood, threads per workgroup, software-pipelined tile
// loop or plain loop); nullptr if unsupported
const void* hmc_kernel_for(int d0, int d1, int layer, int lik, int threads, int pipeline);
// trajectory kernel for layers too wide for register-resident parameters (64 -> 128 -> 1); also
// returns its dynamic LDS size and the floats of private global scratch each workgroup needs
const void* hmc_kernel_wide_for(int d0, int d1, int lik, int threads, size_t* dyn_lds_bytes,
                                size_t* wg_scratch_floats);
hipError_t launch_hmc_kernel(const void* kernel, const KArgs& args, int workgroups, int threads,
                             size_t dyn_lds_bytes, hipStream_t stream);

// small kernels
hipError_t launch_fill_u32(unsigned* p, size_t n, unsigned v, hipStream_t stream);
hipError_t launch_fill_f32(float* p, size_t n, float v, hipStream_t stream);
// status words of a step-operator workspace: cleared on first use only (see prepare_status_kernel);
// launch_clear_status clears a record that has been reported
hipError_t launch_prepare_status(unsigned* status, hipStream_t stream);
hipError_t launch_clear_status(unsigned* status, hipStream_t stream);
// compares the state hashes the workgroups of the last trajectory launch reported (see
// compare_hashes_kernel); status words as described there
hipError_t launch_compare_hashes(const unsigned long long* h, int wgs, int G, unsigned* status,
                                 hipStream_t stream);
hipError_t launch_sample_momentum(uint32_t seed, uint32_t chain_id, uint32_t transition, int n,
                                  float* a, float* b, hipStream_t stream);
hipError_t launch_log_acpt(int n_loss, int n_mom, const float* prev_loss, const float* new_loss,
                           const float* prev_mom, const float* new_mom, const float* grad_cur,
                           float eps, float* out, hipStream_t stream);
hipError_t launch_loss_sums(const float* loss_values, int n, int n_params, float* out2,
                            hipStream_t stream);

}  // namespace bnn
