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
#include "bnn_rng.h"

namespace bnn {

// ================================================================================================
// Lane l = 16 q + n.  Per 16-row tile:
//   GEMM1  A = X tile [16 rows x D0]     lane (n, q) holds row n, k = KS q + s (s < KS = D0 / 4)
//          B = W1 [D0 x 16 c]            read from LDS: k = KS q + s, c = 16 t + n
//          C = pre-activation            lane (n, q) holds rows 4 q + j, c = 16 t + n (bias as C init)
//   GEMM2  A = delta^T = C registers as they are (k-step j <-> rows 4 q + j)
//          B = X tile [4 rows x 16 f]    lane (n, q) holds row 4 q + j, features 32 v + 2 n + u
//          C = dW1^T [16 c x 16 f]       lane (n, q) holds c = 16 t + 4 q + j', f = 32 v + 2 n + u
// ================================================================================================
template <int D0, int D1>
struct MfmaWideLayer {
  static_assert(D0 % 32 == 0 && D1 % 16 == 0, "tiles must divide the layer sizes");
  static constexpr int KS = D0 / 4;
  static constexpr int KQ = KS / 4;  // 16-byte loads of the GEMM1 operand
  static constexpr int NT = D1 / 16;
  static constexpr int FV = D0 / 32;
  static constexpr int FT = 2 * FV;
  static constexpr int oB1 = D0 * D1, oW2 = oB1 + D1, oB2 = oW2 + D1, P = oB2 + 1;
  static constexpr int P_AL = (P + 3) / 4 * 4;
  static constexpr int N_LOADS = KQ + 4 * FV + 1;
  static constexpr float kExp2Scale = -2.88539008177792681472f;  // -2 / ln 2, kernel_helpers.h:37

  f4 dacc[NT][FT];
  float dw2acc[NT];
  float db1acc[NT];
  float db2acc;
  double dl;
  // per step (prepare_step): every lane's part of the layer-2 sum starts from its own share of the
  // constant (sum of w2 - b2) sr2; what the roundings of the 16 shares leave over, and the target
  // times sr2, are added to the finished row sum.  sr2 is the power of two next to 1 / scale, the factor
  // (1 / scale) / sr2 is applied to the finished sum
  float y_0, rho, sr2v, ratio, w2_scale;  // w2_scale = -2 sr2

  struct Tile {
    f4 xa[KQ];
    f2 xb[4][FV];
    float y1;  // target of row 4 q + (n >> 2): lane n sits in bank n >> 2, where that row's sum lands
  };

  __device__ __forceinline__ void zero_acc() {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma unroll
      for (int ft = 0; ft < FT; ++ft) dacc[t][ft] = f4{0.f, 0.f, 0.f, 0.f};
      dw2acc[t] = 0.0f;
      db1acc[t] = 0.0f;
    }
    db2acc = 0.0f;
    dl = 0.0;
  }

  // The pointwise stage works with s = 1 / (1 + 2^t) = (1 + tanh x) / 2 and never forms h = 2 s - 1:
  //   yhat = sum w2 h + b2 = 2 sum w2 s - (sum w2 - b2)        (the constant: once per step, in double)
  //   dw2  = sum g h       = 2 sum g s - sum g                  (add_partials)
  //   1 - h^2 = 4 (s - s^2)                                     (the 4 goes into add_partials)
  // Scaling by a power of two keeps every product of the layer-2 sum exact.
  __device__ __forceinline__ void prepare_step(const float* s_w, const ModelConsts& mc) {
    const int lane = threadIdx.x & 63, n = lane & 15;
    const uint32_t sr2_bits = (__builtin_bit_cast(uint32_t, mc.scale_recp) + 0x00400000u) & 0x7F800000u;
    const float sr2 = __builtin_bit_cast(float, sr2_bits);
    ratio = mc.scale_recp * __builtin_bit_cast(float, 0x7F000000u - sr2_bits);
    // the share of lane n: its hidden units 16 t + n [and b2 in lane 0]; a large constant in one lane
    // would set the rounding grid of that lane's whole sum, and where hidden units saturate the terms
    // take few distinct values, so roundings would repeat from row to row instead of averaging out
    double share = 0.0;
#pragma unroll
    for (int t = 0; t < NT; ++t) share += (double)s_w[oW2 + 16 * t + n];
    if (n == 0) share -= (double)s_w[oB2];
    share *= (double)sr2;
    y_0 = (float)share;
    double rest = share - (double)y_0;
#pragma unroll
    for (int msk = 1; msk < 16; msk <<= 1) rest += shfl_xor_d(rest, msk);
    rho = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, (float)rest)));
    sr2v = sr2;
    w2_scale = -2.0f * sr2;
  }

  // rows past the end read as the last row (their gradient is masked to zero); any alignment
  __device__ __forceinline__ void load_tile_safe(Tile& ti, const StepCtx& cx, int row0, int n,
                                                 int q) const {
    const int last = cx.n - 1;
    const float* ra = cx.X + (size_t)min(row0 + n, last) * D0 + KS * q;
#pragma unroll
    for (int i = 0; i < KQ; ++i) ti.xa[i] = f4{ra[4 * i], ra[4 * i + 1], ra[4 * i + 2], ra[4 * i + 3]};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int rowb = min(row0 + 4 * q + j, last);
      const float* rb = cx.X + (size_t)rowb * D0 + 2 * n;
#pragma unroll
      for (int v = 0; v < FV; ++v) ti.xb[j][v] = f2{rb[32 * v], rb[32 * v + 1]};
    }
    ti.y1 = cx.y[min(row0 + 4 * q + (n >> 2), last)];
  }

  // wait until at most N memory operations are outstanding; the tile's registers are tied to the
  // wait so that nothing that uses them is scheduled above it
  template <int N>
  static __device__ __forceinline__ void wait_tile(Tile& t) {
    static_assert(KQ == 4 && FV == 2, "operand list below is written for D0 = 64");
    asm volatile("s_waitcnt vmcnt(%[cnt])"
                 : "+v"(t.xa[0]), "+v"(t.xa[1]), "+v"(t.xa[2]), "+v"(t.xa[3]), "+v"(t.xb[0][0]),
                   "+v"(t.xb[0][1]), "+v"(t.xb[1][0]), "+v"(t.xb[1][1]), "+v"(t.xb[2][0]),
                   "+v"(t.xb[2][1]), "+v"(t.xb[3][0]), "+v"(t.xb[3][1]), "+v"(t.y1)
                 : [cnt] "n"(N)
                 : "memory");
  }

  // GEMM1 + activation + loss gradient + GEMM2 of one tile
  template <int LIK, bool LAST, bool FULL>
  __device__ __forceinline__ void compute_tile(const Tile& ti, const float* s_w, const StepCtx& cx,
                                               const ModelConsts& mc, int row0, int n, int q) {
    f4 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const float b = s_w[oB1 + 16 * t + n] * kExp2Scale;
      acc[t] = f4{b, b, b, b};
    }
    // W1 operands come from LDS one k-step ahead of the MFMAs that use them (two register sets), so
    // the matrix pipe never waits for an LDS read
    const float* wrow = s_w + (size_t)(KS * q) * D1 + n;
    float bw[2][NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) bw[0][t] = wrow[16 * t];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      if (s + 1 < KS) {
        const float* wk = wrow + (size_t)(s + 1) * D1;
#pragma unroll
        for (int t = 0; t < NT; ++t) bw[(s + 1) & 1][t] = wk[16 * t];
      }
      const float a = ti.xa[s >> 2][s & 3] * kExp2Scale;  // GEMM1 then yields the exp2 argument directly
#pragma unroll
      for (int t = 0; t < NT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, bw[s & 1][t], acc[t], 0, 0, 0);
    }
    // s = 1 / (1 + 2^t) (kernel_helpers.h:34-42 without the small-|x| identity branch, see prepare_step)
    float yh[4] = {y_0, y_0, y_0, y_0};
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const float w2y = s_w[oW2 + 16 * t + n] * w2_scale;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float e = __builtin_amdgcn_exp2f(acc[t][j]);
        const float sg = __builtin_amdgcn_rcpf(1.0f + e);
        acc[t][j] = sg;
        yh[j] = __builtin_fmaf(w2y, sg, yh[j]);
      }
    }
    // scaled residual (y - yhat - b2) / scale of the four rows 4 q + j (mcmc_step_ffma.h:293), in bank
    // j of one register; the loss gradient is computed on that one register
    const float dz = (row16_reduce4(yh[0], yh[1], yh[2], yh[3]) + __builtin_fmaf(ti.y1, sr2v, rho)) * ratio;
    float gz;
    if (LIK == 0) gz = dz * mc.g_scale * __builtin_amdgcn_rcpf(__builtin_fmaf(dz, dz, mc.df));
    else gz = dz * mc.scale_recp;
    float g[4] = {row16_bcast<0>(gz), row16_bcast<1>(gz), row16_bcast<2>(gz), row16_bcast<3>(gz)};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool valid = FULL || (row0 + 4 * q + j < cx.n);
      g[j] = valid ? g[j] : 0.0f;  // mcmc_step_ffma.h:301
      db2acc += g[j];
    }
    if (LAST) {
      const float d4[4] = {row16_bcast<0>(dz), row16_bcast<1>(dz), row16_bcast<2>(dz), row16_bcast<3>(dz)};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const bool valid = FULL || (row0 + 4 * q + j < cx.n);
        if (n == 0 && valid) {
          const int row = row0 + 4 * q + j;
          const float lv = lik_value<LIK>(mc, d4[j]);
          const float prev = cx.ell_prev ? cx.ell_prev[row] : 0.0f;
          if (cx.ell_new) cx.ell_new[row] = lv;
          dl += (double)(lv - prev);
        }
      }
    }
    // GEMM2 operands: u = s - s^2 stays where it is (A), g goes into the rows of x (B); the factors
    // 4 w2[c] of delta are applied once per step to the sums
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float sg = acc[t][j];
        dw2acc[t] = __builtin_fmaf(g[j], sg, dw2acc[t]);
        const float u = __builtin_fmaf(-sg, sg, sg);
        acc[t][j] = u;
        db1acc[t] = __builtin_fmaf(u, g[j], db1acc[t]);
      }
    }
    f2 gx[4][FV];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int v = 0; v < FV; ++v) gx[j][v] = ti.xb[j][v] * g[j];
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
#pragma unroll
        for (int v = 0; v < FV; ++v) {
          dacc[t][2 * v] =
              __builtin_amdgcn_mfma_f32_16x16x4f32(acc[t][j], gx[j][v][0], dacc[t][2 * v], 0, 0, 0);
          dacc[t][2 * v + 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(acc[t][j], gx[j][v][1],
                                                                    dacc[t][2 * v + 1], 0, 0, 0);
        }
      }
    }
  }

  template <int LIK, bool LAST>
  __device__ __forceinline__ void run_tiles(const StepCtx& cx, const ModelConsts& mc,
                                            const float* s_w) {
    const int lane = threadIdx.x & 63, n = lane & 15, q = lane >> 4;
    const int tb = cx.tile_begin, te = cx.tile_end;
    int fast_end = tb;
    if (cx.x_vec_ok && cx.y_vec_ok) fast_end = min(te, cx.n / 16);
    if (fast_end > tb) {
      // loads issued one tile ahead by inline assembly (the compiler neither moves nor waits for
      // them); s_waitcnt vmcnt(N_LOADS) leaves the newer tile in flight
      // every load is a wave-uniform base (SGPRs, scalar arithmetic) plus a fixed 32-bit per-lane
      // offset plus an immediate: no vector instruction is spent on addresses.  One assembly block
      // per tile; its leading s_nop gives the wait states a memory instruction needs after a VALU
      // instruction (a v_readlane reloading a spilled SGPR) wrote one of its SGPR operands -- the
      // compiler does not see the loads inside the block.  Outputs are early-clobber.
      static_assert(KQ == 4 && FV == 2, "operand list below is written for D0 = 64");
      const unsigned oa = (unsigned)((n * D0 + KS * q) * 4);
      const unsigned ob = (unsigned)(((4 * q) * D0 + 2 * n) * 4);
      const unsigned oy = (unsigned)((4 * q + (n >> 2)) * 4);
      auto issue = [&](Tile& t, int tile) {
        tile = tile < fast_end ? tile : fast_end - 1;
        const float* bx = cx.X + (size_t)tile * (16 * D0);
        const float* by = cx.y + (size_t)tile * 16;
        asm volatile(
            "s_nop 4\n\t"
            "global_load_dwordx4 %[a0], %[oa], %[bx]\n\t"
            "global_load_dwordx4 %[a1], %[oa], %[bx] offset:16\n\t"
            "global_load_dwordx4 %[a2], %[oa], %[bx] offset:32\n\t"
            "global_load_dwordx4 %[a3], %[oa], %[bx] offset:48\n\t"
            "global_load_dwordx2 %[b00], %[ob], %[bx]\n\t"
            "global_load_dwordx2 %[b01], %[ob], %[bx] offset:128\n\t"
            "global_load_dwordx2 %[b10], %[ob], %[bx] offset:256\n\t"
            "global_load_dwordx2 %[b11], %[ob], %[bx] offset:384\n\t"
            "global_load_dwordx2 %[b20], %[ob], %[bx] offset:512\n\t"
            "global_load_dwordx2 %[b21], %[ob], %[bx] offset:640\n\t"
            "global_load_dwordx2 %[b30], %[ob], %[bx] offset:768\n\t"
            "global_load_dwordx2 %[b31], %[ob], %[bx] offset:896\n\t"
            "global_load_dword %[yv], %[oy], %[by]"
            : [a0] "=&v"(t.xa[0]), [a1] "=&v"(t.xa[1]), [a2] "=&v"(t.xa[2]), [a3] "=&v"(t.xa[3]),
              [b00] "=&v"(t.xb[0][0]), [b01] "=&v"(t.xb[0][1]), [b10] "=&v"(t.xb[1][0]),
              [b11] "=&v"(t.xb[1][1]), [b20] "=&v"(t.xb[2][0]), [b21] "=&v"(t.xb[2][1]),
              [b30] "=&v"(t.xb[3][0]), [b31] "=&v"(t.xb[3][1]), [yv] "=&v"(t.y1)
            : [oa] "v"(oa), [ob] "v"(ob), [oy] "v"(oy), [bx] "s"(bx), [by] "s"(by)
            : "memory");
      };
      Tile A, B;
      issue(A, tb);
      for (int i = tb; i < fast_end; i += 2) {
        issue(B, i + 1);
        wait_tile<N_LOADS>(A);
        compute_tile<LIK, LAST, true>(A, s_w, cx, mc, i * 16, n, q);
        if (i + 1 < fast_end) {
          issue(A, i + 2);
          wait_tile<N_LOADS>(B);
          compute_tile<LIK, LAST, true>(B, s_w, cx, mc, (i + 1) * 16, n, q);
        }
      }
      wait_tile<0>(A);
      wait_tile<0>(B);
    }
    for (int tile = max(tb, fast_end); tile < te; ++tile) {
      Tile ti;
      load_tile_safe(ti, cx, tile * 16, n, q);
      compute_tile<LIK, LAST, false>(ti, s_w, cx, mc, tile * 16, n, q);
    }
  }

  // add this wave's partial sums into the workgroup record in LDS (canonical parameter numbers);
  // `first` overwrites.  The factor 4 w2[c] left out of delta is applied here, and dw2 is put
  // together from the sums of g s and of g (see prepare_step).
  __device__ __forceinline__ void add_partials(float* red, const float* s_w, bool first) {
    const int lane = threadIdx.x & 63, n = lane & 15, q = lane >> 4;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int c = 16 * t + 4 * q + j;
        const float w2c = 4.0f * s_w[oW2 + c];
#pragma unroll
        for (int ft = 0; ft < FT; ++ft) {
          const int f = 32 * (ft >> 1) + 2 * n + (ft & 1);
          const float v = dacc[t][ft][j] * w2c;
          float* dst = red + f * D1 + c;
          *dst = first ? v : *dst + v;
        }
      }
      // sums over the four row groups q in a fixed order
      float vb = db1acc[t], vw = 2.0f * dw2acc[t] - db2acc;
      vb += __shfl_xor(vb, 16);
      vb += __shfl_xor(vb, 32);
      vw += __shfl_xor(vw, 16);
      vw += __shfl_xor(vw, 32);
      if (q == 0) {
        const int c = 16 * t + n;
        const float b = vb * (4.0f * s_w[oW2 + c]);
        red[oB1 + c] = first ? b : red[oB1 + c] + b;
        red[oW2 + c] = first ? vw : red[oW2 + c] + vw;
      }
    }
    float b = db2acc;  // every lane n of a row group holds the same value
    b += __shfl_xor(b, 16);
    b += __shfl_xor(b, 32);
    double d = dl;  // held by lanes n == 0
    d += shfl_xor_d(d, 16);
    d += shfl_xor_d(d, 32);
    if (lane == 0) {
      red[oB2] = first ? b : red[oB2] + b;
      double* dd = reinterpret_cast<double*>(red + P_AL);
      *dd = first ? d : *dd + d;
    }
  }
};

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
