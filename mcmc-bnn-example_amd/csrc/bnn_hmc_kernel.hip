// Fused HMC trajectory kernel for gfx950 (MI355X).
//
// One persistent launch integrates whole trajectories (and, in MODE_TRANSITIONS, whole HMC
// transitions) for a batch of independent chains.  A chain's rows are shared by G workgroups
// ("chain group"); every workgroup of the group redundantly integrates all P parameters, so only
// the gradient crosses workgroups, once per leapfrog step, through a deterministic two-stage
// reduction: (1) wavefront partials -> LDS slots -> fixed-order sum per workgroup, (2) per-workgroup
// records of flagged packets in global scratch, polled by the readers (no barrier) -> fixed-order
// sum in every workgroup, or, for wide groups, slice by slice in the first workgroups of the group.
//
// What it replaces in the reference: leapfrog_step_kernel (include/mcmc/mcmc_step_ffma.h:154-379),
// the persistent mcmc_step_kernel with its grid barrier (include/mcmc/mcmc_step_tc.h:597-677),
// the momentum lambda, log_acpt_prec, the accept/restore copies, the step-size update and the
// sample store of main_loop (include/mcmc/main.h:204-287).
#include <hip/hip_runtime.h>

#include <type_traits>

#include "bnn_device.h"
#include "bnn_kernel_common.h"
#include "bnn_kernels.h"
#include "bnn_mfma_hybrid_layer.h"
#include "bnn_mfma_layer.h"
#include "bnn_rng.h"

namespace bnn {

// ================================================================================================
// FFMA layer: both contractions on the vector ALU (v_fma_f32).
//
// Lane l = 8 rg + cc (rg = 0..7 row of an 8-row tile pair, cc = 0..7).  Lane (rg, cc) owns hidden
// units c = cc + 8 i (i < HU) for the rows r0 + rg of each 8-row sub-tile: its W1 columns and its
// dW1 accumulators stay in registers for the whole step, the row's features are read once and
// broadcast by the memory system to the 8 lanes that share the row.
// ================================================================================================
template <int D0, int D1>
struct FfmaLayer {
  static_assert(D1 % 8 == 0, "hidden units are dealt to 8 lanes");
  static_assert(D0 % 2 == 0, "feature pairs are read as float2");
  static constexpr int HU = D1 / 8;
  static constexpr int oB1 = D0 * D1, oW2 = oB1 + D1, oB2 = oW2 + D1, P = oB2 + 1;
  static constexpr int P_AL = (P + 3) / 4 * 4;
  static constexpr int TILE_LDS = 0;  // no copy of the tile in LDS

  float w1[D0][HU];
  float b1[HU];
  float w2[HU];
  float b2;
  float dw1[D0][HU];
  float db1[HU];
  float dw2[HU];
  float db2acc;
  double dl;

  struct RowIn {
    float x[D0];
    float yv;
  };

  template <int LIK>
  __device__ __forceinline__ void load_weights(const float* s_w, const ModelConsts&) {
    const int lane = threadIdx.x & 63, cc = lane & 7;
#pragma unroll
    for (int i = 0; i < HU; ++i) {
      const int c = cc + 8 * i;
#pragma unroll
      for (int k = 0; k < D0; ++k) w1[k][i] = s_w[k * D1 + c];
      b1[i] = s_w[oB1 + c];
      w2[i] = s_w[oW2 + c];
    }
    b2 = s_w[oB2];
  }

  __device__ __forceinline__ void prime(const StepCtx&) {}  // nothing is carried from step to step
  __device__ __forceinline__ void zero_acc() {
#pragma unroll
    for (int i = 0; i < HU; ++i) {
#pragma unroll
      for (int k = 0; k < D0; ++k) dw1[k][i] = 0.0f;
      db1[i] = 0.0f;
      dw2[i] = 0.0f;
    }
    db2acc = 0.0f;
    dl = 0.0;
  }

  __device__ __forceinline__ void load_row(RowIn& ri, const StepCtx& cx, int row) const {
    const int r = min(row, cx.n - 1);
    const float* rp = cx.X + (size_t)r * D0;
    if (cx.x_vec_ok) {
#pragma unroll
      for (int k = 0; k < D0; k += 2) {
        const f2 v = *reinterpret_cast<const f2*>(rp + k);
        ri.x[k] = v[0];
        ri.x[k + 1] = v[1];
      }
    } else {
#pragma unroll
      for (int k = 0; k < D0; ++k) ri.x[k] = rp[k];
    }
    ri.yv = cx.y[r];
  }

  template <int LIK, bool LAST>
  __device__ __forceinline__ void compute_row(const RowIn& ri, const StepCtx& cx,
                                              const ModelConsts& mc, int row, int cc) {
    float h[HU];
    // layer 1: FMA chain over k ascending from the bias (mcmc_step_ffma.h:225-255)
#pragma unroll
    for (int i = 0; i < HU; ++i) h[i] = b1[i];
#pragma unroll
    for (int k = 0; k < D0; ++k) {
#pragma unroll
      for (int i = 0; i < HU; ++i) h[i] = __builtin_fmaf(w1[k][i], ri.x[k], h[i]);
    }
    float yh = 0.0f;
#pragma unroll
    for (int i = 0; i < HU; ++i) {
      h[i] = tanh_fwd(h[i]);
      yh = __builtin_fmaf(w2[i], h[i], yh);
    }
    const float yhat = row8_allreduce(yh);
    float diff;
    float g = lik_grad<LIK>(mc, ri.yv - yhat - b2, diff);
    const bool valid = row < cx.n;
    g = valid ? g : 0.0f;
    if (LAST) {
      if (cc == 0 && valid) {
        const float lv = lik_value<LIK>(mc, diff);
        const float prev = cx.ell_prev ? cx.ell_prev[row] : 0.0f;
        if (cx.ell_new) cx.ell_new[row] = lv;
        dl += (double)(lv - prev);
      }
    }
    db2acc += g;
    float delta[HU];
#pragma unroll
    for (int i = 0; i < HU; ++i) {
      dw2[i] = __builtin_fmaf(g, h[i], dw2[i]);
      delta[i] = __builtin_fmaf(-h[i], h[i], 1.0f) * (w2[i] * g);
      db1[i] += delta[i];
    }
#pragma unroll
    for (int k = 0; k < D0; ++k) {
#pragma unroll
      for (int i = 0; i < HU; ++i) dw1[k][i] = __builtin_fmaf(ri.x[k], delta[i], dw1[k][i]);
    }
  }

  template <int LIK, bool LAST>
  __device__ __forceinline__ void run_tiles(const StepCtx& cx, const ModelConsts& mc) {
    const int lane = threadIdx.x & 63, cc = lane & 7, rg = lane >> 3;
    const int row_begin = cx.tile_begin * 16, row_end = min(cx.tile_end * 16, (cx.n + 7) / 8 * 8);
    if (row_begin >= row_end) return;
    RowIn cur, nxt;
    load_row(cur, cx, row_begin + rg);
    for (int r0 = row_begin; r0 < row_end; r0 += 8) {
      const int rn = r0 + 8 < row_end ? r0 + 8 : r0;
      load_row(nxt, cx, rn + rg);  // prefetch
      compute_row<LIK, LAST>(cur, cx, mc, r0 + rg, cc);
      cur = nxt;
    }
  }

  // sum over the 8 row lanes rg (lane bits 3, 4, 5) in a fixed order
  __device__ __forceinline__ float reduce_rg(float v) const {
    v += __shfl_xor(v, 8);
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
    return v;
  }

  // a wave's slot in LDS is indexed by canonical parameter number, the log-likelihood difference behind
  static constexpr int LDS_SLOT = (P_AL + 4 + 31) / 32 * 32;
  static constexpr int DL_INDEX = P_AL;
  static __device__ __forceinline__ int slot_index(int p) { return p; }
  template <int LIK>
  __device__ __forceinline__ float finish(int, float v, const float*) const { return v; }

  template <int LIK>
  __device__ __forceinline__ void write_partials(float* slot, const float*, bool) {
    const int lane = threadIdx.x & 63, cc = lane & 7, rg = lane >> 3;
#pragma unroll
    for (int i = 0; i < HU; ++i) {
      const int c = cc + 8 * i;
#pragma unroll
      for (int k = 0; k < D0; ++k) {
        const float v = reduce_rg(dw1[k][i]);
        if (rg == 0) slot[k * D1 + c] = v;
      }
      const float vb = reduce_rg(db1[i]);
      const float vw = reduce_rg(dw2[i]);
      if (rg == 0) {
        slot[oB1 + c] = vb;
        slot[oW2 + c] = vw;
      }
    }
    const float b = reduce_rg(db2acc);  // every cc lane of a row holds the same g
    double d = dl;                      // held by lanes cc == 0
    d += shfl_xor_d(d, 8);
    d += shfl_xor_d(d, 16);
    d += shfl_xor_d(d, 32);
    if (lane == 0) {
      slot[oB2] = b;
      const uint64_t bits = double_to_bits(d);
      slot[P_AL] = __builtin_bit_cast(float, (uint32_t)bits);
      slot[P_AL + 1] = __builtin_bit_cast(float, (uint32_t)(bits >> 32));
    }
  }
};

// ------------------------------------------------------------------------------------------------
// the kernel
// ------------------------------------------------------------------------------------------------
// Kernel arguments that are needed once per transition or once per launch are not kept in registers
// across the step loop (they would be spilled into lanes of vector registers, which the tile loop has
// none to spare of): COLD(field) reads the field from the kernel-argument segment where it is used.
// The empty assembly statement makes the pointer opaque, so that the load stays where it is written.
__device__ __forceinline__ const __attribute__((address_space(4))) KArgs* cold_args() {
  const __attribute__((address_space(4))) KArgs* p =
      (const __attribute__((address_space(4))) KArgs*)__builtin_amdgcn_kernarg_segment_ptr();
  asm volatile("" : "+s"(p));
  return p;
}
#define COLD(field) (cold_args()->field)

template <class Layer, int LIK, int T>
__global__ __launch_bounds__(T) void hmc_kernel(const KArgs a) {
  constexpr int W = T / 64;
  constexpr int P = Layer::P;
  constexpr int P_AL = Layer::P_AL;
  constexpr int SLOT = (P_AL + 4 + 31) / 32 * 32;  // partial_slot_floats(P)
  constexpr int PPT = (P + T - 1) / T;

  __shared__ float s_w[P_AL];
  __shared__ __align__(16) float s_slots[W][Layer::LDS_SLOT];
  __shared__ double s_red[W];
  __shared__ unsigned long long s_hash[W];
  __shared__ int s_progress[W];
  // a wave's copy of the tile it is working on (the hybrid MFMA layer only)
  __shared__ __align__(16) float s_tile[W][Layer::TILE_LDS > 0 ? Layer::TILE_LDS : 4];
  // kept out of registers while a trajectory runs (a thread only ever touches the entries of the
  // parameters it owns, so no barrier guards them): the accepted position and its gradient, the
  // start momentum of the running transition, and the thread's state hash
  __shared__ float s_wc[PPT * T], s_gc[PPT * T], s_m0[PPT * T];
  __shared__ unsigned long long s_hacc[T];
  __shared__ int s_flag[2];  // by step parity: cleared by a thread that abandoned a wait
  // stage 2: the sums over the records (own array: the waves' slots may still be being read by stage 1
  // of a slower wave), the reducers' per-wave slice sums, the log-likelihood difference
  __shared__ float s_sum[P_AL];
  __shared__ float s_red2[W][32];
  __shared__ double s_dl;

  // ---- which chain group, which rank inside it ----
  int lin = blockIdx.x;
  if (a.xcd_map) {
    const int per_xcd = gridDim.x >> 3;
    lin = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  }
  const int group = lin / a.G, rank = lin - group * a.G;
  if (a.debug_xcc && threadIdx.x == 0) {
    // XCC_ID hardware register (id 20), bits 3:0
    a.debug_xcc[blockIdx.x] = __builtin_amdgcn_s_getreg((3 << 11) | 20);
  }
  if (group >= a.n_groups) return;
  int chain = a.chain_base + group;
  if (a.chain_wrap > 0 && chain >= a.chain_wrap) chain -= a.chain_wrap;
  const int window = a.fixed_window >= 0 ? a.fixed_window : chain / a.chains_per_window;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, kept in an SGPR

  StepCtx cx;
  cx.X = a.X + (size_t)window * a.x_stride;
  cx.y = a.y + (size_t)window * a.y_stride;
  cx.n = a.n;
  cx.x_vec_ok = a.x_vec_ok != 0;
  cx.y_vec_ok = a.y_vec_ok != 0;
  {
    // The rows go to the waves in equal contiguous runs of tiles, the remainder spread evenly along
    // the run order.  Waves w and w + W / 2 share a SIMD: they take neighbouring runs, so that when the
    // tile count does not divide no SIMD gets two of the longer runs while another gets two short ones.
    const int pos = W == 8 ? ((wave & 3) * 2 + (wave >> 2)) : wave;
    const int gw = rank * W + pos, GW = a.G * W;
    cx.tile_begin = (int)((long)a.n_tiles * gw / GW);
    cx.tile_end = (int)((long)a.n_tiles * (gw + 1) / GW);
  }
  cx.ell_prev = nullptr;
  cx.ell_new = nullptr;
  // waves w and w + W / 2 sit on the same SIMD (waves are dealt to the four SIMDs in turn)
  cx.progress = (a.balance && W == 8) ? s_progress : nullptr;
  cx.wave = wave;
  cx.partner = wave ^ (W / 2);
  cx.tile_lds = s_tile[wave];

  const ModelConsts mc = a.mc;
  // records of flagged packets (8 bytes per parameter), two per workgroup (by step parity)
  unsigned long long* part_base = reinterpret_cast<unsigned long long*>(a.partials) + (size_t)group * 2 * a.G * SLOT;
  unsigned bar_epoch = 0;
  int buf = 0;

  // ---- parameters owned by this thread: p = tid + i T ----
  float w[PPT], m[PPT], g[PPT];
  float eps;
  int t0 = 0, sel = 0, nacc = 0;
  const bool trans = a.mode == MODE_TRANSITIONS;
#pragma unroll
  for (int i = 0; i < PPT; ++i) {
    const int p = tid + i * T;
    w[i] = m[i] = g[i] = 0.0f;
    s_wc[tid + i * T] = s_gc[tid + i * T] = s_m0[tid + i * T] = 0.0f;
    if (p < P) {
      if (trans) {
        s_wc[p] = a.st_w[(size_t)chain * a.st_stride + p];
        s_gc[p] = a.st_g[(size_t)chain * a.st_stride + p];
      } else {
        const size_t o = (size_t)group * a.in_stride + p;
        w[i] = a.w_in ? a.w_in[o] : 0.0f;
        m[i] = a.m_in ? a.m_in[o] : 0.0f;
        g[i] = a.g_in ? a.g_in[o] : 0.0f;
      }
    }
  }
  if (trans) {
    eps = a.st_eps[chain];
    t0 = a.st_t[chain];
    sel = a.st_sel[chain];
    nacc = a.st_nacc[chain];
  } else {
    eps = a.eps_in;
  }

  Layer layer;
  cx.back = leapfrog_walks_back(0, a.L);
  cx.back_next = cx.back;
  layer.prime(cx);  // the first tiles of the first gradient evaluation
  bool ok = true;
  // optional per-phase cycle accounting (thread 0 of each workgroup)
  unsigned long long ph[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  unsigned long long tstamp = 0;
  const bool prof = a.debug_phase != nullptr;
#define BNN_PHASE(k)                                        \
  if (prof) {                                               \
    const unsigned long long now_ = __builtin_readcyclecounter(); \
    ph[k] += now_ - tstamp;                                 \
    tstamp = now_;                                          \
  }
  unsigned long long clk0 = 0, rt0 = 0;
  if (prof) {
    tstamp = clk0 = __builtin_readcyclecounter();
    rt0 = __builtin_amdgcn_s_memrealtime();
  }
  const int n_outer = trans ? a.n_trans : 1;
  double dl_total = 0.0;
  s_hacc[tid] = 0;  // state hash, see fold_hash

  for (int it = 0; it < n_outer && ok; ++it) {
    const uint32_t t = (uint32_t)(t0 + it);
    float* ell_cur = nullptr;
    float* ell_prop = nullptr;
    if (trans) {
      // momentum resampling (main.h:207-216); the start state is the last accepted one
#pragma unroll
      for (int i = 0; i < PPT; ++i) {
        const int p = tid + i * T;
        if (p < P) {
          m[i] = rng_normal(COLD(seed), (uint32_t)chain + COLD(rng_id_base), STREAM_MOMENTUM, t, (uint64_t)p);
          s_m0[p] = m[i];
          w[i] = s_wc[p];
          g[i] = s_gc[p];
        }
      }
      ell_cur = (sel ? COLD(ell1) : COLD(ell0)) + (size_t)chain * COLD(ell_stride);
      ell_prop = (sel ? COLD(ell0) : COLD(ell1)) + (size_t)chain * COLD(ell_stride);
    } else {
      ell_prop = COLD(ell_out) ? COLD(ell_out) + (size_t)group * COLD(ell_stride) : nullptr;
    }

    for (int s = 0; s < a.L && ok; ++s) {
      // indices and addresses that depend on the thread index are recomputed every step (see
      // opaque_tid): hoisted out of this loop they would occupy registers across the tile loop
      const int tid = opaque_tid();
      // ---- leapfrog update (mcmc_step_ffma.h:106-112): half kick on the first step ----
      const float ek = s == 0 ? eps * 0.5f : eps;
#pragma unroll
      for (int i = 0; i < PPT; ++i) {
        const int p = tid + i * T;
        if (p < P) {
          m[i] = __builtin_fmaf(ek, g[i], m[i]);
          w[i] = __builtin_fmaf(eps, m[i], w[i]);
          s_w[p] = w[i];
        }
      }
      if ((tid & 63) == 0) s_progress[wave] = 0;
      const unsigned epoch = bar_epoch + 1;  // the steps of this launch from 1
      if (tid == 0) s_flag[epoch & 1] = 1;
      __syncthreads();
      BNN_PHASE(0)  // update + sync
      layer.template load_weights<LIK>(s_w, mc);
      layer.zero_acc();
      BNN_PHASE(1)  // operand fetch from LDS
      const bool last = s == a.L - 1;
      cx.back = leapfrog_walks_back(s, a.L);
      cx.back_next = leapfrog_walks_back(last ? 0 : s + 1, a.L);
      if (last) {
        cx.ell_prev = ell_cur;
        cx.ell_new = ell_prop;
        layer.template run_tiles<LIK, true>(cx, mc);
      } else {
        layer.template run_tiles<LIK, false>(cx, mc);
      }
      BNN_PHASE(2)  // tile loop
      layer.template write_partials<LIK>(s_slots[wave], s_w, last);
      __syncthreads();
      BNN_PHASE(3)  // wave partials -> LDS + sync
      // ---- stage 1: fixed-order sum over this workgroup's waves -> the workgroup's record of flagged
      //      packets (see st_packet); the padding up to P_AL is written too, so that every 16-byte column
      //      a reader polls is complete ----
      ++bar_epoch;
      unsigned long long* my_part = part_base + ((size_t)buf * a.G + rank) * SLOT;
      if (rank != a.debug_drop_rank) {
        // (all reads of the waves' slots are issued before the first addition: one LDS latency, not W)
        float sv[PPT][W];
#pragma unroll
        for (int i = 0; i < PPT; ++i) {
          const int idx = Layer::slot_index(min(tid + i * T, P - 1));
#pragma unroll
          for (int wv = 0; wv < W; ++wv) sv[i][wv] = s_slots[wv][idx];
        }
        keep_together(sv);
#pragma unroll
        for (int i = 0; i < PPT; ++i) {
          const int p = tid + i * T;
          if (p < P_AL) {
            float v = sv[i][0];
#pragma unroll
            for (int wv = 1; wv < W; ++wv) v += sv[i][wv];
            st_packet(my_part + p, p < P ? layer.template finish<LIK>(p, v, s_w) : 0.0f, epoch);
          }
        }
        if (last && tid == 0) {
          double d = 0.0;
#pragma unroll
          for (int wv = 0; wv < W; ++wv) {
            const uint64_t bits = ((uint64_t)__builtin_bit_cast(uint32_t, s_slots[wv][Layer::DL_INDEX + 1]) << 32) |
                                  __builtin_bit_cast(uint32_t, s_slots[wv][Layer::DL_INDEX]);
            d += bits_to_double(bits);
          }
          const uint64_t bits = double_to_bits(d);
          st_packet(my_part + P_AL, __builtin_bit_cast(float, (uint32_t)bits), epoch);
          st_packet(my_part + P_AL + 1, __builtin_bit_cast(float, (uint32_t)(bits >> 32)), epoch);
        }
      }
      BNN_PHASE(4)  // stage 1 + global store
      BNN_PHASE(5)  // (no barrier: the records are polled)
      const unsigned long long* grp_part = part_base + (size_t)buf * a.G * SLOT;
      bool fine = true;  // cleared by a thread whose wait was abandoned
      // the log-likelihood difference of the records, in record order per lane and a fixed tree over
      // the lanes (last step only; one wave)
      auto sum_dl = [&]() {
        const int lane = tid & 63;
        double d = 0.0;
        for (int r = lane; r < a.G; r += 64) {
          const float lo = wait_packet(grp_part + (size_t)r * SLOT + P_AL, epoch, a.status, a.spin_limit, fine);
          const float hi = wait_packet(grp_part + (size_t)r * SLOT + P_AL + 1, epoch, a.status, a.spin_limit, fine);
          d += bits_to_double(((uint64_t)__builtin_bit_cast(uint32_t, hi) << 32) |
                              __builtin_bit_cast(uint32_t, lo));
        }
#pragma unroll
        for (int msk = 1; msk < 64; msk <<= 1) d += shfl_xor_d(d, msk);
        return d;
      };
      if (!a.two_phase) {
        // ---- stage 2 (small groups): every workgroup adds the G records.  A thread takes 16-byte
        //      columns (two parameters) of the records, eight loads in flight, records in ascending
        //      order, polling until all of them are this step's; the prior gradient is added as block 0
        //      does in the reference (mcmc_step_ffma.h:144) ----
        constexpr int NCOL = P_AL / 2;
        for (int col = tid; col < NCOL; col += T) {
          float v0 = 0.0f, v1 = 0.0f;
          const unsigned long long* src = grp_part + 2 * col;
          for (int r0 = 0; r0 < a.G; r0 += 8) {
            f4 t8[8];
            const unsigned long long* p8[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) p8[k] = src + (size_t)min(r0 + k, a.G - 1) * SLOT;
            wait_packets4x8(t8, p8, a.G - r0, epoch, a.status, a.spin_limit, fine);
#pragma unroll
            for (int k = 0; k < 8; ++k)
              if (r0 + k < a.G) {  // wave-uniform condition
                v0 += t8[k][0];
                v1 += t8[k][2];
              }
          }
          s_sum[2 * col] = v0;
          s_sum[2 * col + 1] = v1;
        }
        if (last && wave == W - 1) {
          const double d = sum_dl();
          if ((tid & 63) == 0) s_dl = d;
        }
      } else {
        // ---- stage 2 (large groups), in two phases.  Phase 1: workgroup `rank` < ceil(P / SL) reduces
        //      the SL-parameter slice [SL rank, SL rank + SL) over all G records: thread (record lane
        //      rl = tid / CS, 16-byte column c = tid % CS, CS = SL / 2) adds records rl, rl + T / CS, ...
        //      in order, the record lanes of a wave are added by a fixed xor tree and the waves in order
        //      through LDS; the totals go out as flagged packets.  Phase 2: everyone polls the totals. ----
        unsigned long long* tot_all =
            reinterpret_cast<unsigned long long*>(a.totals) + (size_t)group * TOTALS_COPIES * SLOT;
        // one copy per 32 workgroups of the group (a group of 32 polls its single copy as it stands)
        const int copies = min(TOTALS_COPIES, a.G >> 5);
        const unsigned long long* tot = tot_all + (size_t)(rank % copies) * SLOT;  // the copy this rank polls
        // The wider the group, the narrower the slices and the more reducers: what bounds the first
        // hand-off is the time one workgroup needs to pull its slice of every record through its own
        // memory path (G x 256 bytes for a 32-parameter slice), and a poll that comes too early repeats
        // all of it.  From 64 workgroups on the slices are 16 parameters wide (one 128-byte line of every
        // record, 61 reducers), below that 32 (31 reducers).  Measured, ms per 1000 steps of one chain,
        // slices of 32 / 16 / 8 parameters: G = 256: 9.31 / 9.25 / 9.47, G = 128: 11.84 / 11.56 / 12.12,
        // G = 64: 17.01 / 16.75 / -.
        const int CSr = a.G >= 64 ? 8 : 16;  // 16-byte columns per slice
        const int SL = 2 * CSr;                                  // parameters per slice
        const int n_red = (P_AL + SL - 1) / SL;
        const bool reducer = rank < n_red;
        auto reduce_slice = [&](auto cs_c, auto nb_c) {
          constexpr int CS = decltype(cs_c)::value;
          constexpr int RL = T / CS;                   // record lanes of a workgroup
          constexpr int NB = decltype(nb_c)::value;    // records per thread and poll
          const int c = tid & (CS - 1), rl = tid / CS;
          const bool col_ok = 2 * CS * rank + 2 * c < P_AL;  // P_AL is even: a column is whole or absent
          const unsigned long long* src = grp_part + 2 * CS * rank + 2 * c;
          float v0 = 0.0f, v1 = 0.0f;
          for (int r0 = rl; r0 < a.G; r0 += NB * RL) {
            f4 t8[8];
            const unsigned long long* p8[8];
            int valid = 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
              p8[k] = src + (size_t)min(r0 + RL * (k < NB ? k : 0), a.G - 1) * SLOT;
              if (k < NB && r0 + RL * k < a.G) valid = k + 1;
            }
            wait_packets4x8<NB>(t8, p8, col_ok ? valid : 0, epoch, a.status, a.spin_limit, fine);
#pragma unroll
            for (int k = 0; k < NB; ++k)
              if (k < valid) {
                v0 += t8[k][0];
                v1 += t8[k][2];
              }
          }
          // the record lanes of a wave (lanes that differ in the bits above the column index)
#pragma unroll
          for (int msk = CS; msk < 64; msk <<= 1) {
            v0 += __shfl_xor(v0, msk);
            v1 += __shfl_xor(v1, msk);
          }
          if ((tid & 63) < CS) {
            s_red2[wave][2 * c] = v0;
            s_red2[wave][2 * c + 1] = v1;
          }
        };
        if (reducer) {
          // as many loads in flight per thread as it has records (at most eight a poll)
          const int per_thread = (a.G * CSr + T - 1) / T;
          using std::integral_constant;
          if (CSr == 8) {
            if (per_thread <= 2) reduce_slice(integral_constant<int, 8>{}, integral_constant<int, 2>{});
            else if (per_thread <= 4) reduce_slice(integral_constant<int, 8>{}, integral_constant<int, 4>{});
            else reduce_slice(integral_constant<int, 8>{}, integral_constant<int, 8>{});
          } else {
            if (per_thread <= 2) reduce_slice(integral_constant<int, 16>{}, integral_constant<int, 2>{});
            else if (per_thread <= 4) reduce_slice(integral_constant<int, 16>{}, integral_constant<int, 4>{});
            else reduce_slice(integral_constant<int, 16>{}, integral_constant<int, 8>{});
          }
        }
        __syncthreads();
        static_assert(T >= 32 * TOTALS_COPIES, "one thread per parameter of the slice and copy");
        if (reducer && tid < SL * copies && SL * rank + (tid & (SL - 1)) < P_AL && rank != a.debug_drop_rank) {
          const int pp = tid & (SL - 1), copy = tid / SL;
          float rv[1][W];
#pragma unroll
          for (int wv = 0; wv < W; ++wv) rv[0][wv] = s_red2[wv][pp];
          keep_together(rv);
          float x = rv[0][0];
#pragma unroll
          for (int wv = 1; wv < W; ++wv) x += rv[0][wv];
          st_packet(tot_all + (size_t)copy * SLOT + SL * rank + pp, x, epoch);
        }
        if (last && rank == n_red - 1 && wave == W - 1) {
          const double d = sum_dl();
          if ((tid & 63) == 0) {
            const uint64_t bits = double_to_bits(d);
            for (int copy = 0; copy < copies; ++copy) {
              unsigned long long* tc = tot_all + (size_t)copy * SLOT;
              st_packet(tc + P_AL, __builtin_bit_cast(float, (uint32_t)bits), epoch);
              st_packet(tc + P_AL + 1, __builtin_bit_cast(float, (uint32_t)(bits >> 32)), epoch);
            }
          }
        }
        // (the totals cannot be there before the reducers have seen every record: a workgroup that has
        // nothing to reduce waits about a microsecond before its first poll instead of loading the
        // memory system with polls that must fail)
        if (!reducer) __builtin_amdgcn_s_sleep(48);
        // a thread polls one 16-byte column (two packets) of the totals: one memory round trip
        constexpr int NCOL = P_AL / 2;
        for (int col = tid; col < NCOL; col += T) {
          const f4 t4 = wait_packets4(tot + 2 * col, epoch, a.status, a.spin_limit, fine);
          s_sum[2 * col] = t4[0];
          s_sum[2 * col + 1] = t4[2];
        }
        if (last && tid == 0) {
          const float lo = wait_packet(tot + P_AL, epoch, a.status, a.spin_limit, fine);
          const float hi = wait_packet(tot + P_AL + 1, epoch, a.status, a.spin_limit, fine);
          s_dl = bits_to_double(((uint64_t)__builtin_bit_cast(uint32_t, hi) << 32) |
                                __builtin_bit_cast(uint32_t, lo));
        }
      }
      if (!fine) s_flag[epoch & 1] = 0;
      __syncthreads();
      ok = s_flag[epoch & 1] != 0;
      if (!ok) break;
#pragma unroll
      for (int i = 0; i < PPT; ++i) {
        const int p = tid + i * T;
        if (p < P) g[i] = prior_grad(mc, w[i]) + s_sum[p];
      }
      if (last) dl_total = s_dl;
      buf ^= 1;
      BNN_PHASE(6)  // stage 2
    }
    if (!ok) break;

    if (trans) {
      // ---- log accept ratio (kernel_helpers.h:163-175): sum over rows is dl_total; prior and
      //      kinetic terms summed here in a fixed order ----
      double part = 0.0;
#pragma unroll
      for (int i = 0; i < PPT; ++i) {
        const int p = tid + i * T;
        if (p < P) {
          const float dp = prior_logp(mc, w[i]) - prior_logp(mc, s_wc[p]);
          const float nm = __builtin_fmaf(eps * 0.5f, g[i], m[i]);  // final half kick
          const float m0 = s_m0[p];
          float kt = m0 * m0;
          kt = __builtin_fmaf(-nm, nm, kt);
          part += (double)dp + (double)(0.5f * kt);
        }
      }
#pragma unroll
      for (int msk = 1; msk < 64; msk <<= 1) part += shfl_xor_d(part, msk);
      __syncthreads();
      if ((tid & 63) == 0) s_red[wave] = part;
      __syncthreads();
      double tot = dl_total;
#pragma unroll
      for (int wv = 0; wv < W; ++wv) tot += s_red[wv];
      const float la = (float)tot;
      // ---- Metropolis decision (main.h:235-265) ----
      const float lu = rng_log_uniform(COLD(seed), (uint32_t)chain + COLD(rng_id_base), t);
      const bool acc = lu < la;
      if (acc) {
#pragma unroll
        for (int i = 0; i < PPT; ++i) {
          s_wc[tid + i * T] = w[i];
          s_gc[tid + i * T] = g[i];
        }
        sel ^= 1;
        ++nacc;
      }
      // ---- step-size adaptation (main.h:267-276); a non-finite ratio counts as minus infinity ----
      if ((int)t < COLD(adapt_steps)) {
        const float laf = (la == la) ? la : -__builtin_inff();
        const float lmin = laf < 0.0f ? laf : 0.0f;
        const float adj = lmin < COLD(log_target) ? COLD(dec_adj) : COLD(inc_adj);
        eps = eps + eps * adj;
      }
      // what this workgroup holds after the transition goes into its state hash
      {
        unsigned long long hacc = s_hacc[tid];
#pragma unroll
        for (int i = 0; i < PPT; ++i) hacc = fold_hash(hacc, s_wc[tid + i * T], s_gc[tid + i * T]);
        s_hacc[tid] = fold_hash(hacc, la, eps) + (unsigned long long)nacc;
      }
      if (rank == 0) {
        // ---- sample store (main.h:277-283) and traces ----
        if ((int)t >= COLD(burn_in) && (int)t - COLD(burn_in) < COLD(n_samples)) {
          float* dst = COLD(samples) + ((size_t)chain * COLD(n_samples) + ((int)t - COLD(burn_in))) * P;
#pragma unroll
          for (int i = 0; i < PPT; ++i) {
            const int p = tid + i * T;
            if (p < P) dst[p] = s_wc[p];
          }
        }
        if (tid == 0 && (int)t < COLD(trace_len)) {
          COLD(tr_log_acpt)[(size_t)chain * COLD(trace_len) + t] = la;
          COLD(tr_accept)[(size_t)chain * COLD(trace_len) + t] = acc ? 1 : 0;
          COLD(tr_eps)[(size_t)chain * COLD(trace_len) + t] = eps;
        }
      }
    }
  }

  if (prof && tid == 0) {
    BNN_PHASE(7)  // transition epilogue
#pragma unroll
    for (int k = 0; k < 8; ++k) COLD(debug_phase)[(size_t)blockIdx.x * 10 + k] = ph[k];
    // shader-clock ticks and 100 MHz real-time ticks of the whole launch: their ratio is the clock
    COLD(debug_phase)[(size_t)blockIdx.x * 10 + 8] = __builtin_readcyclecounter() - clk0;
    COLD(debug_phase)[(size_t)blockIdx.x * 10 + 9] = __builtin_amdgcn_s_memrealtime() - rt0;
  }
#undef BNN_PHASE
  if (!ok) return;
  if (COLD(rank_hash)) {
    unsigned long long hacc = s_hacc[tid];
    if (!trans) {
#pragma unroll
      for (int i = 0; i < PPT; ++i) hacc = fold_hash(fold_hash(hacc, w[i], g[i]), m[i], eps);
    }
    publish_hash(hacc, s_hash, W, COLD(rank_hash) + lin, rank == COLD(debug_perturb_hash_rank));
  }
  // ---- write back ----
  if (rank == 0) {
    if (trans) {
#pragma unroll
      for (int i = 0; i < PPT; ++i) {
        const int p = tid + i * T;
        if (p < P) {
          COLD(st_w)[(size_t)chain * COLD(st_stride) + p] = s_wc[p];
          COLD(st_g)[(size_t)chain * COLD(st_stride) + p] = s_gc[p];
        }
      }
      if (tid == 0) {
        COLD(st_eps)[chain] = eps;
        COLD(st_t)[chain] = t0 + COLD(n_trans);
        COLD(st_sel)[chain] = sel;
        COLD(st_nacc)[chain] = nacc;
      }
    } else {
      double psum = 0.0;
#pragma unroll
      for (int i = 0; i < PPT; ++i) {
        const int p = tid + i * T;
        if (p < P) {
          const size_t o = (size_t)group * COLD(out_stride) + p;
          const float lp = prior_logp(mc, w[i]);
          if (COLD(w_out)) COLD(w_out)[o] = w[i];
          if (COLD(m_out)) COLD(m_out)[o] = m[i];
          if (COLD(g_out)) COLD(g_out)[o] = g[i];
          if (COLD(g_zero)) COLD(g_zero)[o] = 0.0f;
          if (COLD(prior_out)) COLD(prior_out)[o] = lp;
          psum += (double)lp;
        }
      }
      if (COLD(sums_out)) {
#pragma unroll
        for (int msk = 1; msk < 64; msk <<= 1) psum += shfl_xor_d(psum, msk);
        __syncthreads();
        if ((tid & 63) == 0) s_red[wave] = psum;
        __syncthreads();
        if (tid == 0) {
          double tot = 0.0;
#pragma unroll
          for (int wv = 0; wv < W; ++wv) tot += s_red[wv];
          COLD(sums_out)[(size_t)group * 2 + 0] = dl_total;
          COLD(sums_out)[(size_t)group * 2 + 1] = tot;
        }
      }
    }
  }
}

#undef COLD

// ------------------------------------------------------------------------------------------------
// host-side launcher
// ------------------------------------------------------------------------------------------------
template <class Layer, int LIK, int T>
static const void* kernel_ptr() {
  return reinterpret_cast<const void*>(&hmc_kernel<Layer, LIK, T>);
}

const void* hmc_kernel_for(int d0, int d1, int layer, int lik, int threads, int pipeline) {
  if (d0 != 22 || d1 != 40) return nullptr;
  using MP = MfmaLayer<22, 40, 1>;
  using MS = MfmaLayer<22, 40, 0>;
  using MA = MfmaLayer<22, 40, 2>;
  using MH = MfmaHybridLayer<22, 40>;
  using F = FfmaLayer<22, 40>;
  if (layer == 0 && pipeline == 4) {
    // hidden units 32 .. 39 on 4x4 blocks (bnn_mfma_hybrid_layer.h): prefetched loop, 512 threads only
    if (threads == 512) return lik == 0 ? kernel_ptr<MH, 0, 512>() : kernel_ptr<MH, 1, 512>();
  } else if (layer == 0 && pipeline == 2) {
    // The prefetched loop is built for 512 threads only.  Its loads are issued from inline assembly
    // and land in their registers long after the compiler believes them written: with fewer than
    // 256 VGPRs per thread (768 or 1024 threads) the kernel spills, and a register that is spilled or
    // re-used while its load is still in flight is corrupted.  The build checks that this kernel (and
    // the wide-layer kernel, which loads the same way) has no spills.
    if (threads == 512) return lik == 0 ? kernel_ptr<MA, 0, 512>() : kernel_ptr<MA, 1, 512>();
  } else if (layer == 0 && pipeline == 1) {
    if (threads == 512) return lik == 0 ? kernel_ptr<MP, 0, 512>() : kernel_ptr<MP, 1, 512>();
    if (threads == 256) return lik == 0 ? kernel_ptr<MP, 0, 256>() : kernel_ptr<MP, 1, 256>();
  } else if (layer == 0) {
    if (threads == 1024) return lik == 0 ? kernel_ptr<MS, 0, 1024>() : kernel_ptr<MS, 1, 1024>();
    if (threads == 768) return lik == 0 ? kernel_ptr<MS, 0, 768>() : kernel_ptr<MS, 1, 768>();
    if (threads == 512) return lik == 0 ? kernel_ptr<MS, 0, 512>() : kernel_ptr<MS, 1, 512>();
    if (threads == 256) return lik == 0 ? kernel_ptr<MS, 0, 256>() : kernel_ptr<MS, 1, 256>();
  } else if (layer == 1) {
    if (threads == 256) return lik == 0 ? kernel_ptr<F, 0, 256>() : kernel_ptr<F, 1, 256>();
  }
  return nullptr;
}

hipError_t launch_hmc_kernel(const void* kernel, const KArgs& args, int workgroups, int threads,
                             size_t dyn_lds_bytes, hipStream_t stream) {
  KArgs a = args;
  void* params[] = {&a};
  return hipLaunchKernel(kernel, dim3(workgroups), dim3(threads), params, dyn_lds_bytes, stream);
}

}  // namespace bnn
