// Trajectory kernel for wide layers (64 -> 128 -> 1, P = 8449 parameters): the same algorithm as
// bnn_hmc_kernel.hip -- fused leapfrog update, forward, loss, backward, deterministic two-stage
// gradient reduction, and in MODE_TRANSITIONS the whole HMC transition -- laid out for a parameter
// vector that no longer fits registers: weights, momentum and gradient of the trajectory live in LDS
// (3 x 33 KB), the accepted state and the start momentum in a per-workgroup global scratch record,
// and the GEMM1 weight operand is read from LDS as it is consumed.  Both contractions run on
// v_mfma_f32_16x16x4_f32 with no padding (64 and 128 are multiples of the tile sizes).
//
// Reference counterparts as in bnn_hmc_kernel.hip (include/mcmc/mcmc_step_ffma.h:154-427,
// include/mcmc/mcmc_step_tc.h:597-677, include/mcmc/main.h:204-287).
#include <hip/hip_runtime.h>

#include "bnn_device.h"
#include "bnn_kernel_common.h"
#include "bnn_kernels.h"
#include "bnn_mfma_wide_layer.h"
#include "bnn_rng.h"

namespace bnn {

// ------------------------------------------------------------------------------------------------
template <class Layer, int LIK, int T>
__global__ __launch_bounds__(T) void hmc_kernel_wide(const KArgs a) {
  constexpr int W = T / 64;
  constexpr int P = Layer::P;
  constexpr int P_AL = Layer::P_AL;
  constexpr int SLOT = (P_AL + 4 + 31) / 32 * 32;  // partial_slot_floats(P)

  extern __shared__ __align__(16) float s_dyn[];
  float* s_w = s_dyn;             // position of the trajectory (GEMM1 / pointwise operand)
  float* s_m = s_w + P_AL;        // momentum
  float* s_g = s_m + P_AL;        // gradient at s_w
  float* s_red = s_g + P_AL;      // workgroup partial record (SLOT floats, the last four hold a double)
  __shared__ double s_wsum[W];
  __shared__ unsigned long long s_hash[W];
  __shared__ int s_flag;

  int lin = blockIdx.x;
  if (a.xcd_map) {
    const int per_xcd = gridDim.x >> 3;
    lin = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  }
  const int group = lin / a.G, rank = lin - group * a.G;
  if (group >= a.n_groups) return;
  int chain = a.chain_base + group;
  if (a.chain_wrap > 0 && chain >= a.chain_wrap) chain -= a.chain_wrap;
  const int window = a.fixed_window >= 0 ? a.fixed_window : chain / a.chains_per_window;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  StepCtx cx;
  cx.X = a.X + (size_t)window * a.x_stride;
  cx.y = a.y + (size_t)window * a.y_stride;
  cx.n = a.n;
  cx.x_vec_ok = a.x_vec_ok != 0;
  cx.y_vec_ok = a.y_vec_ok != 0;
  {
    const int gw = rank * W + wave, GW = a.G * W;
    cx.tile_begin = (int)((long)a.n_tiles * gw / GW);
    cx.tile_end = (int)((long)a.n_tiles * (gw + 1) / GW);
  }
  cx.ell_prev = nullptr;
  cx.ell_new = nullptr;

  const ModelConsts mc = a.mc;
  float* part_base = a.partials + (size_t)group * 2 * a.G * SLOT;
  unsigned* counter = a.barrier + (size_t)group * BARRIER_STRIDE_WORDS;
  unsigned bar_epoch = 0;
  int buf = 0;

  const bool trans = a.mode == MODE_TRANSITIONS;
  // accepted position, its gradient and the start momentum of the running transition: private to
  // this workgroup, in global memory (touched once per transition)
  float* wc = a.wg_scratch + (size_t)blockIdx.x * 3 * P_AL;
  float* gc = wc + P_AL;
  float* m0 = gc + P_AL;
  float eps;
  int t0 = 0, sel = 0, nacc = 0;
  if (trans) {
    for (int p = tid; p < P; p += T) {
      wc[p] = a.st_w[(size_t)chain * a.st_stride + p];
      gc[p] = a.st_g[(size_t)chain * a.st_stride + p];
    }
    eps = a.st_eps[chain];
    t0 = a.st_t[chain];
    sel = a.st_sel[chain];
    nacc = a.st_nacc[chain];
  } else {
    for (int p = tid; p < P; p += T) {
      const size_t o = (size_t)group * a.in_stride + p;
      s_w[p] = a.w_in ? a.w_in[o] : 0.0f;
      s_m[p] = a.m_in ? a.m_in[o] : 0.0f;
      s_g[p] = a.g_in ? a.g_in[o] : 0.0f;
    }
    eps = a.eps_in;
  }

  Layer layer;
  bool ok = true;
  const int n_outer = trans ? a.n_trans : 1;
  double dl_total = 0.0;
  unsigned long long hacc = 0;  // state hash, see fold_hash

  for (int it = 0; it < n_outer && ok; ++it) {
    const uint32_t t = (uint32_t)(t0 + it);
    float* ell_cur = nullptr;
    float* ell_prop = nullptr;
    if (trans) {
      // momentum resampling (main.h:207-216); the start state is the last accepted one.  Every
      // thread owns the parameters p = tid, tid + T, ... throughout.
      for (int p = tid; p < P; p += T) {
        const float z = rng_normal(a.seed, (uint32_t)chain + a.rng_id_base, STREAM_MOMENTUM, t, (uint64_t)p);
        m0[p] = z;
        s_m[p] = z;
        s_w[p] = wc[p];
        s_g[p] = gc[p];
      }
      ell_cur = (sel ? a.ell1 : a.ell0) + (size_t)chain * a.ell_stride;
      ell_prop = (sel ? a.ell0 : a.ell1) + (size_t)chain * a.ell_stride;
    } else {
      ell_prop = a.ell_out ? a.ell_out + (size_t)group * a.ell_stride : nullptr;
    }

    for (int s = 0; s < a.L && ok; ++s) {
      // ---- leapfrog update (mcmc_step_ffma.h:106-112): half kick on the first step ----
      const float ek = s == 0 ? eps * 0.5f : eps;
      for (int p = tid; p < P; p += T) {
        const float mm = __builtin_fmaf(ek, s_g[p], s_m[p]);
        s_m[p] = mm;
        s_w[p] = __builtin_fmaf(eps, mm, s_w[p]);
      }
      __syncthreads();
      layer.zero_acc();
      layer.prepare_step(s_w, mc);
      const bool last = s == a.L - 1;
      if (last) {
        cx.ell_prev = ell_cur;
        cx.ell_new = ell_prop;
        layer.template run_tiles<LIK, true>(cx, mc, s_w);
      } else {
        layer.template run_tiles<LIK, false>(cx, mc, s_w);
      }
      // ---- stage 1: the waves add their partials to the workgroup record one after the other ----
      for (int wv = 0; wv < W; ++wv) {
        if (wave == wv) layer.add_partials(s_red, s_w, wv == 0);
        __syncthreads();
      }
      float* my_part = part_base + ((size_t)buf * a.G + rank) * SLOT;
      for (int p = tid; p < P_AL + 2; p += T)
        if (p < P || p >= P_AL) st_agent(my_part + p, s_red[p]);
      ok = group_barrier(counter, a.G, rank, ++bar_epoch, a.status, a.spin_limit, &s_flag,
                         rank != a.debug_drop_rank);
      if (!ok) break;
      const float* grp_part = part_base + (size_t)buf * a.G * SLOT;
      if (!a.two_phase) {
        // ---- stage 2 (up to 64 workgroups per chain): every workgroup adds the G records in rank
        //      order, seeded with the prior gradient (mcmc_step_ffma.h:144).  A thread takes 16-byte
        //      columns of the records, eight loads in flight ----
        for (int col = tid; col < P_AL / 4; col += T) {
          f4 v = {0.f, 0.f, 0.f, 0.f};
          const float* src = grp_part + 4 * col;
          for (int r0 = 0; r0 < a.G; r0 += 8) {
            f4 t8[8];
            const float* p8[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) p8[k] = src + (size_t)min(r0 + k, a.G - 1) * SLOT;
            ld_agent4x8(t8, p8);
#pragma unroll
            for (int k = 0; k < 8; ++k)
              if (r0 + k < a.G) v += t8[k];
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int p = 4 * col + e;
            if (p < P) s_g[p] = prior_grad(mc, s_w[p]) + v[e];
          }
        }
        __syncthreads();  // the columns are not the parameters a thread owns in the update loops
        if (last) {
          double d = 0.0;
          for (int r = 0; r < a.G; ++r) {
            const float lo = ld_agent(grp_part + (size_t)r * SLOT + P_AL);
            const float hi = ld_agent(grp_part + (size_t)r * SLOT + P_AL + 1);
            d += bits_to_double(((uint64_t)__builtin_bit_cast(uint32_t, hi) << 32) |
                                __builtin_bit_cast(uint32_t, lo));
          }
          dl_total = d;
        }
      } else {
        // ---- stage 2 (more than 64 workgroups per chain), in two phases: reading all G records in
        //      every workgroup would move G * G * 34 KB per step.  Phase 1: workgroup `rank` reduces
        //      the 32-parameter slices rank, rank + G, ... -- one 128-byte line of every record each --
        //      over all G records: thread (record lane rl = tid / 8, 16-byte column c = tid % 8) adds
        //      records rl, rl + T/8, ... in order, the record lanes of a wave are added by a fixed xor
        //      tree and the waves in order through LDS.  Phase 2, once every slice is stored: everyone
        //      reads the totals. ----
        float* tot = a.totals + (size_t)group * SLOT;
        constexpr int RL = T / 8;                  // record lanes of a workgroup
        constexpr int N_SLICE = (P + 31) / 32;
        float* s_x = s_red;                        // free: this step's record has been published
        for (int sl = rank; sl < N_SLICE; sl += a.G) {
          const int c = tid & 7, rl = tid >> 3;
          const float* src = grp_part + 32 * sl + 4 * c;
          f4 v = {0.f, 0.f, 0.f, 0.f};
          for (int r0 = rl; r0 < a.G; r0 += 8 * RL) {
            f4 t8[8];
            const float* p8[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) p8[k] = src + (size_t)min(r0 + RL * k, a.G - 1) * SLOT;
            ld_agent4x8(t8, p8);
#pragma unroll
            for (int k = 0; k < 8; ++k)
              if (r0 + RL * k < a.G) v += t8[k];
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float x = v[e];
            x += __shfl_xor(x, 8);
            x += __shfl_xor(x, 16);
            x += __shfl_xor(x, 32);
            v[e] = x;
          }
          __syncthreads();  // the previous slice's sums have been read
          if ((tid & 63) < 8) *reinterpret_cast<f4*>(&s_x[32 * wave + 4 * c]) = v;
          __syncthreads();
          if (tid < 32 && 32 * sl + tid < P) {
            float x = s_x[tid];
#pragma unroll
            for (int wv = 1; wv < W; ++wv) x += s_x[32 * wv + tid];
            st_agent(tot + 32 * sl + tid, x);
          }
        }
        if (last && rank == a.G - 1 && wave == W - 1) {
          const int lane = tid & 63;
          double d = 0.0;
          for (int r = lane; r < a.G; r += 64) {
            const float lo = ld_agent(grp_part + (size_t)r * SLOT + P_AL);
            const float hi = ld_agent(grp_part + (size_t)r * SLOT + P_AL + 1);
            d += bits_to_double(((uint64_t)__builtin_bit_cast(uint32_t, hi) << 32) |
                                __builtin_bit_cast(uint32_t, lo));
          }
#pragma unroll
          for (int msk = 1; msk < 64; msk <<= 1) d += shfl_xor_d(d, msk);
          if (lane == 0) {
            const uint64_t bits = double_to_bits(d);
            st_agent(tot + P_AL, __builtin_bit_cast(float, (uint32_t)bits));
            st_agent(tot + P_AL + 1, __builtin_bit_cast(float, (uint32_t)(bits >> 32)));
          }
        }
        // every workgroup has slices to announce (G <= number of slices), everybody waits for all
        ok = reducer_barrier(counter, a.G, true, rank, bar_epoch, a.status, a.spin_limit, &s_flag,
                             rank != a.debug_drop_rank);
        if (!ok) break;
        for (int p = tid; p < P; p += T) s_g[p] = prior_grad(mc, s_w[p]) + ld_agent(tot + p);
        if (last) {
          const float lo = ld_agent(tot + P_AL);
          const float hi = ld_agent(tot + P_AL + 1);
          dl_total = bits_to_double(((uint64_t)__builtin_bit_cast(uint32_t, hi) << 32) |
                                    __builtin_bit_cast(uint32_t, lo));
        }
      }
      buf ^= 1;
    }
    if (!ok) break;

    if (trans) {
      // ---- log accept ratio (kernel_helpers.h:163-175): rows in dl_total; prior and kinetic terms
      //      here, in a fixed order ----
      double part = 0.0;
      for (int p = tid; p < P; p += T) {
        const float dp = prior_logp(mc, s_w[p]) - prior_logp(mc, wc[p]);
        const float nm = __builtin_fmaf(eps * 0.5f, s_g[p], s_m[p]);  // final half kick
        float kt = m0[p] * m0[p];
        kt = __builtin_fmaf(-nm, nm, kt);
        part += (double)dp + (double)(0.5f * kt);
      }
#pragma unroll
      for (int msk = 1; msk < 64; msk <<= 1) part += shfl_xor_d(part, msk);
      __syncthreads();
      if ((tid & 63) == 0) s_wsum[wave] = part;
      __syncthreads();
      double tot = dl_total;
#pragma unroll
      for (int wv = 0; wv < W; ++wv) tot += s_wsum[wv];
      const float la = (float)tot;
      // ---- Metropolis decision (main.h:235-265) ----
      const float lu = rng_log_uniform(a.seed, (uint32_t)chain + a.rng_id_base, t);
      const bool acc = lu < la;
      if (acc) {
        for (int p = tid; p < P; p += T) {
          wc[p] = s_w[p];
          gc[p] = s_g[p];
        }
        sel ^= 1;
        ++nacc;
      }
      // ---- step-size adaptation (main.h:267-276); a non-finite ratio counts as minus infinity ----
      if ((int)t < a.adapt_steps) {
        const float laf = (la == la) ? la : -__builtin_inff();
        const float lmin = laf < 0.0f ? laf : 0.0f;
        const float adj = lmin < a.log_target ? a.dec_adj : a.inc_adj;
        eps = eps + eps * adj;
      }
      // what this workgroup holds after the transition goes into its state hash
      for (int p = tid; p < P; p += T) hacc = fold_hash(hacc, wc[p], gc[p]);
      hacc = fold_hash(hacc, la, eps) + (unsigned long long)nacc;
      if (rank == 0) {
        // ---- sample store (main.h:277-283) and traces ----
        if ((int)t >= a.burn_in && (int)t - a.burn_in < a.n_samples) {
          float* dst = a.samples + ((size_t)chain * a.n_samples + ((int)t - a.burn_in)) * P;
          for (int p = tid; p < P; p += T) dst[p] = wc[p];
        }
        if (tid == 0 && (int)t < a.trace_len) {
          a.tr_log_acpt[(size_t)chain * a.trace_len + t] = la;
          a.tr_accept[(size_t)chain * a.trace_len + t] = acc ? 1 : 0;
          a.tr_eps[(size_t)chain * a.trace_len + t] = eps;
        }
      }
    }
  }

  if (!ok) return;
  if (a.rank_hash) {
    if (!trans)
      for (int p = tid; p < P; p += T) hacc = fold_hash(fold_hash(hacc, s_w[p], s_g[p]), s_m[p], eps);
    publish_hash(hacc, s_hash, W, a.rank_hash + lin, rank == a.debug_perturb_hash_rank);
  }
  if (rank == 0) {
    if (trans) {
      for (int p = tid; p < P; p += T) {
        a.st_w[(size_t)chain * a.st_stride + p] = wc[p];
        a.st_g[(size_t)chain * a.st_stride + p] = gc[p];
      }
      if (tid == 0) {
        a.st_eps[chain] = eps;
        a.st_t[chain] = t0 + a.n_trans;
        a.st_sel[chain] = sel;
        a.st_nacc[chain] = nacc;
      }
    } else {
      double psum = 0.0;
      for (int p = tid; p < P; p += T) {
        const size_t o = (size_t)group * a.out_stride + p;
        const float lp = prior_logp(mc, s_w[p]);
        if (a.w_out) a.w_out[o] = s_w[p];
        if (a.m_out) a.m_out[o] = s_m[p];
        if (a.g_out) a.g_out[o] = s_g[p];
        if (a.g_zero) a.g_zero[o] = 0.0f;
        if (a.prior_out) a.prior_out[o] = lp;
        psum += (double)lp;
      }
      if (a.sums_out) {
#pragma unroll
        for (int msk = 1; msk < 64; msk <<= 1) psum += shfl_xor_d(psum, msk);
        __syncthreads();
        if ((tid & 63) == 0) s_wsum[wave] = psum;
        __syncthreads();
        if (tid == 0) {
          double tot = 0.0;
#pragma unroll
          for (int wv = 0; wv < W; ++wv) tot += s_wsum[wv];
          a.sums_out[(size_t)group * 2 + 0] = dl_total;
          a.sums_out[(size_t)group * 2 + 1] = tot;
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
const void* hmc_kernel_wide_for(int d0, int d1, int lik, int threads, size_t* dyn_lds_bytes,
                                size_t* wg_scratch_floats) {
  if (d0 != 64 || d1 != 128 || threads != 256) return nullptr;
  using L = MfmaWideLayer<64, 128>;
  if (dyn_lds_bytes) *dyn_lds_bytes = (size_t)(3 * L::P_AL + partial_slot_floats(L::P)) * sizeof(float);
  if (wg_scratch_floats) *wg_scratch_floats = (size_t)3 * L::P_AL;
  return lik == 0 ? reinterpret_cast<const void*>(&hmc_kernel_wide<L, 0, 256>)
                  : reinterpret_cast<const void*>(&hmc_kernel_wide<L, 1, 256>);
}

}  // namespace bnn
