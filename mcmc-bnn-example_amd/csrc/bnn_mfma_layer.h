// The MFMA layer of the 22 -> 40 -> 1 trajectory kernel: both contractions of a 16-row tile on the FP32
// matrix instructions (16x16x4 tiles and 4x4x1 blocks), the pointwise stage between them, the tile loops
// and the wave's partial sums.  In a header of its own
// so that the tile-ceiling probe (tile_ceiling.hip) times exactly the code the kernel runs.
#pragma once

#include <hip/hip_runtime.h>

#include "bnn_device.h"
#include "bnn_kernel_common.h"

namespace bnn {

// Constant operand slots of the MFMA layer: `one` reads (1, 0) at offsets j * D0 (j < 4), `zero` reads
// (0, 0); lanes holding the appended constant-one feature or tile padding point here.
template <int D0>
struct AugTable {
  float one[3 * D0 + 4];
  float zero[3 * D0 + 4];
};
template <int D0>
constexpr AugTable<D0> make_aug_table() {
  AugTable<D0> t{};
  for (int j = 0; j < 4; ++j) t.one[j * D0] = 1.0f;
  return t;
}
__device__ const AugTable<22> k_aug_table_22 = make_aug_table<22>();
template <int D0>
__device__ __forceinline__ const AugTable<D0>* aug_table();
template <>
__device__ __forceinline__ const AugTable<22>* aug_table<22>() {
  return &k_aug_table_22;
}

// ================================================================================================
// MFMA layer: GEMM1 and most of GEMM2 on v_mfma_f32_16x16x4_f32, the rest of GEMM2 on
// v_mfma_f32_4x4x1_16B_f32 (same flops per cycle, but sixteen independent 4x4 outer products: no
// padding of the seven feature columns that a second 16-wide tile would leave half empty).
//
// Lane l = 16 q + n (q = 0..3, n = 0..15; n = 4 cb + jj).  A 16-row tile is processed as
//   GEMM1   A = X_aug tile  [16 rows x K]    lane (n, q) holds row n, k = KS q + s      (s < KS)
//           B = W1_aug      [K x 16 c]       lane (n, q) holds k = KS q + s, c = 16 t + n
//           C = pre-act     [16 rows x 16 c] lane (n, q) holds rows 4 q + j, c = 16 t + n
//   GEMM2e  A = delta^T     [16 c x 4 rows]  = C layout of GEMM1 reused as is (k-step j <-> rows
//                                              4 q + j): no shuffle between the two GEMMs
//           B = X tile      [4 rows x 16 f]  lane (n, q) holds row 4 q + j, feature n      (f < 16)
//           C = dW1^T       [16 c x 16 f]    lane (n, q) holds c = 16 t + 4 q + i, f = n
//   GEMM2f  sixteen blocks b = 4 q + cb per instruction, one instruction per (t, j, fb):
//           A block = delta of row 4 q + j, c = 16 t + 4 cb + i     (the same register as above)
//           B block = X_aug of row 4 q + j, f = 16 + 2 jj + fb      (lane (n, q), any cb)
//           D block = dW1_aug^T partial of row group q: vgpr i, lane (n, q): c = 16 t + 4 cb + i,
//                     f = 16 + 2 jj + fb; the four row groups are added once per step
// X_aug appends a constant-one feature (index D0) so that b1 rides in GEMM1 and db1 falls out of
// GEMM2; the contraction index of GEMM1 is permuted so that every lane reads contiguous floats.
// ================================================================================================
template <int D0, int D1, int PIPE>
struct MfmaLayer {
  static_assert(D0 % 2 == 0, "feature pairs are read as float2");
  static constexpr int KS = (D0 + 1 + 3) / 4;  // k-steps of GEMM1 (one more feature: the bias)
  static_assert(KS % 2 == 0, "k-steps are read in pairs");
  static constexpr int KP = KS / 2;
  static constexpr int NT = (D1 + 15) / 16;  // hidden tiles
  static_assert(D0 > 16 && D0 + 2 <= 24, "features 16 .. D0 + 1 go through the 4x4 blocks");
  static constexpr int oB1 = D0 * D1, oW2 = oB1 + D1, oB2 = oW2 + D1, P = oB2 + 1;
  static constexpr int P_AL = (P + 3) / 4 * 4;
  static constexpr int TILE_LDS = 0;  // no copy of the tile in LDS

  // The activation is carried as the logistic value s = 1 / (1 + 2^t) = (h + 1) / 2 and h = tanh is
  // never formed: the layer-2 dot, the layer-2 weight gradient and 1 - h^2 = 4 s (1 - s) are all
  // affine in s or products of s, and the constants move into per-step operands (one VALU
  // instruction less per hidden value and row).
  float w1b[KS][NT];   // W1_aug scaled by -2/ln 2: GEMM1 yields the exp2 argument t of the activation
  float w2g[NT];       // -2 w2[c] k2: the layer-2 dot yields r = (y - yhat - b2) k2, where k2 is the power
                       // of two next to k = 1/scale^2 (Gaussian: r k / k2 is the per-row loss gradient)
                       // or k = 1/scale (Student-t: r k / k2 is the scaled residual).  A power of two
                       // keeps the coefficients exact: the dot cancels from terms of size |w2| k to a
                       // residual thousands of times smaller, and a rounding error in a coefficient
                       // would be the same in every row and add up over the rows instead of averaging out
  float k2v;           // k2 (the same in every lane): the target y enters as y k2 after the row sums
  float y_0;           // where this lane's partial sum starts: its share of the constant (sum_c w2[c] - b2) k2
  float rho;           // what the roundings of the 16 shares leave over (the same in every lane)
  float ratio;         // k / k2 (exact)
  // sums over rows of s (1 - s) g' x_aug, g' = g k2 / k (Gaussian) or g (Student-t):
  f4 dacc_e[NT];       //   features 0 .. 15
  f4 dacc_f[NT][2];    //   features 16 .. D0 + 1, partial over the rows of row group q
  float dw2s[NT];      // sum over rows of g' s
                       // (in the lanes of the padded hidden units, where s is exactly 1/2, this is half the
                       // sum over rows of g', added in the very order of the other lanes' sums: dw2 =
                       // 2 (dw2s - that) is then exactly zero where every s is 1/2 -- all weights zero,
                       // the reference's start)
  double dl;

  struct TileIn {
    f2 xa[KP];   // GEMM1 operand
    float xe[4]; // GEMM2e operand: feature n of rows 4 q + j
    f2 xf[4];    // GEMM2f operand: features 16 + 2 jj, 17 + 2 jj of rows 4 q + j
    float y1;    // target of row 4 q + (n >> 2): lane n sits in bank n >> 2, where that row's sum lands
  };

  static constexpr float kExp2Scale = -2.88539008177792681472f;  // -2 / ln 2, kernel_helpers.h:37

  template <int LIK>
  __device__ __forceinline__ void load_weights(const float* s_w, const ModelConsts& mc) {
    const int lane = opaque_tid() & 63, n = lane & 15, q = lane >> 4;
    const float k = LIK == 1 ? mc.scale_recp * mc.scale_recp : mc.scale_recp;
    // the power of two next to k, and its reciprocal
    const uint32_t k2_bits = (__builtin_bit_cast(uint32_t, k) + 0x00400000u) & 0x7F800000u;
    const float k2 = __builtin_bit_cast(float, k2_bits);
    ratio = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(
        int, k * __builtin_bit_cast(float, 0x7F000000u - k2_bits))));
    double w2lane = 0.0;  // sum of the layer-2 weights of this lane's hidden units
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int c = 16 * t + n;
      const bool cv = c < D1;
      const int cc = cv ? c : 0;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        // (one unconditional read per slot: a read under a lane mask would be waited for on its own)
        const int kk = KS * q + s;
        const float v = s_w[kk < D0 ? kk * D1 + cc : oB1 + cc];  // kk == D0: the bias row; beyond: padding
        w1b[s][t] = cv && kk <= D0 ? v * kExp2Scale : 0.0f;
      }
      const float w2c = cv ? s_w[oW2 + cc] : 0.0f;
      w2lane += (double)w2c;
      w2g[t] = -2.0f * w2c * k2;
    }
    // Each lane's partial sum starts from its own share of the constant, k2 (sum of its w2 [- b2 in
    // lane 0]), so that it stays of the size of k2 sum w2 h (the tanh form's): a large constant in one
    // lane would set the rounding grid of that lane's whole sum, and where hidden units saturate (s
    // exactly 0 or 1) the terms take few distinct values, so roundings repeat from row to row instead of
    // averaging out.  What the 16 roundings of the shares leave over (exactly known in double) is
    // added after the row sum, together with the target.
    const double share = (w2lane - (n == 0 ? (double)s_w[oB2] : 0.0)) * (double)k2;
    y_0 = (float)share;
    const double rest = row16_allreduce_d(share - (double)y_0);
    rho = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, (float)rest)));
    k2v = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, k2)));
  }

  __device__ __forceinline__ void zero_acc() {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      dacc_e[t] = f4{0.f, 0.f, 0.f, 0.f};
      dacc_f[t][0] = f4{0.f, 0.f, 0.f, 0.f};
      dacc_f[t][1] = f4{0.f, 0.f, 0.f, 0.f};
      dw2s[t] = 0.0f;
    }
    dl = 0.0;
  }

  // the constant GEMM2f operand of lanes whose feature pair starts at or beyond D0: (1, 0) for the
  // appended constant-one feature, else (0, 0)
  static __device__ __forceinline__ f2 const_f(int jj) { return f2{16 + 2 * jj == D0 ? 1.0f : 0.0f, 0.0f}; }

  // rows past the end read as the last row (their gradient is masked to zero); any alignment
  __device__ __forceinline__ void load_tile_safe(TileIn& ti, const StepCtx& cx, int row0, int n,
                                                 int q) const {
    const int last = cx.n - 1;
    const int rowa = min(row0 + n, last);
    const float* ra = cx.X + (size_t)rowa * D0;
#pragma unroll
    for (int i = 0; i < KP; ++i) {
      const int k0 = KS * q + 2 * i;
      const int kc = k0 < D0 ? k0 : D0 - 2;
      f2 v = f2{ra[kc], ra[kc + 1]};
      if (k0 >= D0) v = f2{k0 == D0 ? 1.0f : 0.0f, 0.0f};
      ti.xa[i] = v;
    }
    const int jj = n & 3;
    const int f0 = 16 + 2 * jj;
    const int fc = f0 < D0 ? f0 : D0 - 2;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int rowb = min(row0 + 4 * q + j, last);
      const float* rb = cx.X + (size_t)rowb * D0;
      ti.xe[j] = rb[n];
      ti.xf[j] = f0 < D0 ? f2{rb[fc], rb[fc + 1]} : const_f(jj);
    }
    ti.y1 = cx.y[min(row0 + 4 * q + (n >> 2), last)];
  }

  // ordinary loads of a full, aligned tile through per-lane pointers (the plain and the software-
  // pipelined loop).  Lanes whose operand slot is the constant-one feature or padding read it from a
  // small constant table through a pointer with stride zero, so no select sits between a load and its use.
  struct PlainPtrs {
    const float* pa;        // row n, k = KS q of tile 0
    const float* pa_last0;  // last k-pair: real data, or the (1, 0) constant in lane group q = 3
    unsigned sa_last;
    const float* pe;        // rows 4 q + j, feature n
    const float* pf0;       // rows 4 q + j, features 16 + 2 jj ..: real data or constants
    unsigned sf;
    const float* py;        // row 4 q + (n >> 2)
    int tb;
  };
  __device__ __forceinline__ PlainPtrs plain_ptrs(const StepCtx& cx, int tb, int n, int q) const {
    const AugTable<D0>* aug = aug_table<D0>();
    const size_t tile_floats = (size_t)16 * D0;
    PlainPtrs p;
    p.tb = tb;
    p.pa = cx.X + (size_t)n * D0 + KS * q;
    const bool a_const = KS * q + 2 * (KP - 1) >= D0;
    p.pa_last0 = a_const ? aug->one : p.pa + (size_t)tb * tile_floats + 2 * (KP - 1);
    p.sa_last = a_const ? 0u : (unsigned)tile_floats;
    p.pe = cx.X + (size_t)(4 * q) * D0 + n;
    const int jj = n & 3;
    const bool f_const = 16 + 2 * jj >= D0;
    p.pf0 = f_const ? (16 + 2 * jj == D0 ? aug->one : aug->zero)
                    : cx.X + ((size_t)tb * 16 + 4 * q) * D0 + 16 + 2 * jj;
    p.sf = f_const ? 0u : (unsigned)tile_floats;
    p.py = cx.y + 4 * q + (n >> 2);
    return p;
  }
  __device__ __forceinline__ void load_plain(TileIn& ti, const PlainPtrs& p, int tile) const {
    const size_t tile_floats = (size_t)16 * D0;
    const float* ra = p.pa + (size_t)tile * tile_floats;
#pragma unroll
    for (int i = 0; i < KP - 1; ++i) ti.xa[i] = *reinterpret_cast<const f2*>(ra + 2 * i);
    const unsigned rel = (unsigned)(tile - p.tb);
    ti.xa[KP - 1] = *reinterpret_cast<const f2*>(p.pa_last0 + (size_t)rel * p.sa_last);
    const float* re = p.pe + (size_t)tile * tile_floats;
    const float* rf = p.pf0 + (size_t)rel * p.sf;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      ti.xe[j] = re[j * D0];
      ti.xf[j] = *reinterpret_cast<const f2*>(rf + j * D0);
    }
    ti.y1 = p.py[(size_t)tile * 16];
  }

  // ---- the stages of a tile ----
  // B: GEMM1, pre-activations (bias included through the constant-one feature)
  __device__ __forceinline__ void gemm1(const f2 (&xa)[KP], f4 (&acc)[NT]) const {
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < KP; ++i) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(xa[i][0], w1b[2 * i][t], acc[t], 0, 0, 0);
#pragma unroll
      for (int t = 0; t < NT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(xa[i][1], w1b[2 * i + 1][t], acc[t], 0, 0, 0);
    }
  }

  // C: activation, layer-2 dot, per-row loss gradient, layer-2 weight gradient, the GEMM2
  // operands.  acc arrives as the exp2 argument t = -2 x / ln 2 of s = 1 / (1 + 2^t), tanh(x) = 2 s - 1
  // (kernel_helpers.h:34-42 without its small-|x| identity branch, which changes the value by less
  // than 1.5e-7), and leaves as s (1 - s) = (1 - tanh^2) / 4.  The factors g (per row) and 4 w2[c]
  // (per hidden unit) of delta = (1 - h^2) w2[c] g (kernel_helpers.h:43, mcmc_step_ffma.h:323) are
  // applied to the other GEMM2 operand (g x_aug: 12 products per tile) and once per step to the GEMM2
  // result.  The padded hidden units (zero weights: s = 1/2) carry 1/4, so the constant-one column
  // of GEMM2 delivers sum(g) / 4 = db2 / 4 in row c = D1 for free.
  template <int LIK, bool LAST, bool FULL>
  __device__ __forceinline__ void pointwise(f4 (&acc)[NT], const TileIn& ti, float (&ge)[4], f2 (&gf)[4],
                                            const StepCtx& cx, const ModelConsts& mc, int row0, int n,
                                            int q) {
    float yh[4] = {y_0, y_0, y_0, y_0};
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float e = __builtin_amdgcn_exp2f(acc[t][j]);
        const float sg = __builtin_amdgcn_rcpf(1.0f + e);
        acc[t][j] = sg;
        yh[j] = __builtin_fmaf(w2g[t], sg, yh[j]);
      }
    }
    // (y - yhat - b2) k2 of the four rows 4 q + j, in bank j of one register; the loss gradient
    // (Gaussian: that value itself, its factor k / k2 is applied to the sums once per step;
    // Student-t: mcmc_step_ffma.h:293-301) is computed on that one register
    const float rz = row16_reduce4(yh[0], yh[1], yh[2], yh[3]) + __builtin_fmaf(ti.y1, k2v, rho);
    float gz = rz, dz = rz;
    if (LIK == 0) {
      dz = rz * ratio;
      gz = dz * mc.g_scale * __builtin_amdgcn_rcpf(__builtin_fmaf(dz, dz, mc.df));
    }
    float g[4];
    if (!FULL) {
      g[0] = row16_bcast<0>(gz);
      g[1] = row16_bcast<1>(gz);
      g[2] = row16_bcast<2>(gz);
      g[3] = row16_bcast<3>(gz);
#pragma unroll
      for (int j = 0; j < 4; ++j) g[j] = row0 + 4 * q + j < cx.n ? g[j] : 0.0f;  // mcmc_step_ffma.h:301
    }
    if (LAST) {
      const float d4[4] = {row16_bcast<0>(dz), row16_bcast<1>(dz), row16_bcast<2>(dz), row16_bcast<3>(dz)};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const bool valid = FULL || (row0 + 4 * q + j < cx.n);
        if (n == 0 && valid) {
          const float diff = LIK == 1 ? d4[j] * (ratio * mc.scale) : d4[j];
          const int row = row0 + 4 * q + j;
          const float lv = lik_value<LIK>(mc, diff);
          const float prev = cx.ell_prev ? cx.ell_prev[row] : 0.0f;
          if (cx.ell_new) cx.ell_new[row] = lv;
          dl += (double)(lv - prev);
        }
      }
    }
    if (FULL) {
      // every consumer of g takes it straight out of its bank of gz (a DPP operand), so the four
      // values are never copied into registers of their own
      consume_g(acc, gz, ti, ge, gf);
    } else {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
#pragma unroll
        for (int j = 0; j < 4; ++j) dw2s[t] = __builtin_fmaf(g[j], acc[t][j], dw2s[t]);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        ge[j] = ti.xe[j] * g[j];
        gf[j] = ti.xf[j] * g[j];
      }
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float sg = acc[t][j];
        acc[t][j] = __builtin_fmaf(-sg, sg, sg);
      }
    }
  }

  // dw2s[t] += g_j s[t][j] and (ge, gf)[j] = g_j (xe, xf)[j], where g_j sits in bank j of gz and is
  // read through a DPP row broadcast (no builtin pairs a broadcast with a multiply-add, hence the
  // assembly; the leading s_nop keeps the DPP reads two wait states behind the instruction that
  // wrote gz).  The order of the additions into dw2s[t] is j = 0, 1, 2, 3.
  __device__ __forceinline__ void consume_g(const f4 (&s)[NT], float gz, const TileIn& ti, float (&ge)[4],
                                            f2 (&gf)[4]) {
    static_assert(NT == 3, "operand lists are written for three hidden tiles");
#define BNN_BC(j) " row_newbcast:" #j " row_mask:0xf bank_mask:0xf\n\t"
    asm("s_nop 1\n\t"
        "v_fmac_f32_dpp %[d0], %[g], %[s00]" BNN_BC(0)
        "v_fmac_f32_dpp %[d1], %[g], %[s10]" BNN_BC(0)
        "v_fmac_f32_dpp %[d2], %[g], %[s20]" BNN_BC(0)
        "v_fmac_f32_dpp %[d0], %[g], %[s01]" BNN_BC(4)
        "v_fmac_f32_dpp %[d1], %[g], %[s11]" BNN_BC(4)
        "v_fmac_f32_dpp %[d2], %[g], %[s21]" BNN_BC(4)
        "v_fmac_f32_dpp %[d0], %[g], %[s02]" BNN_BC(8)
        "v_fmac_f32_dpp %[d1], %[g], %[s12]" BNN_BC(8)
        "v_fmac_f32_dpp %[d2], %[g], %[s22]" BNN_BC(8)
        "v_fmac_f32_dpp %[d0], %[g], %[s03]" BNN_BC(12)
        "v_fmac_f32_dpp %[d1], %[g], %[s13]" BNN_BC(12)
        "v_fmac_f32_dpp %[d2], %[g], %[s23] row_newbcast:12 row_mask:0xf bank_mask:0xf"
        : [d0] "+v"(dw2s[0]), [d1] "+v"(dw2s[1]), [d2] "+v"(dw2s[2])
        : [g] "v"(gz), [s00] "v"(s[0][0]), [s01] "v"(s[0][1]), [s02] "v"(s[0][2]), [s03] "v"(s[0][3]),
          [s10] "v"(s[1][0]), [s11] "v"(s[1][1]), [s12] "v"(s[1][2]), [s13] "v"(s[1][3]),
          [s20] "v"(s[2][0]), [s21] "v"(s[2][1]), [s22] "v"(s[2][2]), [s23] "v"(s[2][3]));
    float f00, f01, f10, f11, f20, f21, f30, f31;
    asm("s_nop 1\n\t"
        "v_mul_f32_dpp %[e0], %[g], %[x0]" BNN_BC(0)
        "v_mul_f32_dpp %[a0], %[g], %[p0]" BNN_BC(0)
        "v_mul_f32_dpp %[b0], %[g], %[r0]" BNN_BC(0)
        "v_mul_f32_dpp %[e1], %[g], %[x1]" BNN_BC(4)
        "v_mul_f32_dpp %[a1], %[g], %[p1]" BNN_BC(4)
        "v_mul_f32_dpp %[b1], %[g], %[r1]" BNN_BC(4)
        "v_mul_f32_dpp %[e2], %[g], %[x2]" BNN_BC(8)
        "v_mul_f32_dpp %[a2], %[g], %[p2]" BNN_BC(8)
        "v_mul_f32_dpp %[b2], %[g], %[r2]" BNN_BC(8)
        "v_mul_f32_dpp %[e3], %[g], %[x3]" BNN_BC(12)
        "v_mul_f32_dpp %[a3], %[g], %[p3]" BNN_BC(12)
        "v_mul_f32_dpp %[b3], %[g], %[r3] row_newbcast:12 row_mask:0xf bank_mask:0xf"
        : [e0] "=&v"(ge[0]), [e1] "=&v"(ge[1]), [e2] "=&v"(ge[2]), [e3] "=&v"(ge[3]), [a0] "=&v"(f00),
          [b0] "=&v"(f01), [a1] "=&v"(f10), [b1] "=&v"(f11), [a2] "=&v"(f20), [b2] "=&v"(f21),
          [a3] "=&v"(f30), [b3] "=&v"(f31)
        : [g] "v"(gz), [x0] "v"(ti.xe[0]), [x1] "v"(ti.xe[1]), [x2] "v"(ti.xe[2]), [x3] "v"(ti.xe[3]),
          [p0] "v"(ti.xf[0][0]), [r0] "v"(ti.xf[0][1]), [p1] "v"(ti.xf[1][0]), [r1] "v"(ti.xf[1][1]),
          [p2] "v"(ti.xf[2][0]), [r2] "v"(ti.xf[2][1]), [p3] "v"(ti.xf[3][0]), [r3] "v"(ti.xf[3][1]));
#undef BNN_BC
    gf[0] = f2{f00, f01};
    gf[1] = f2{f10, f11};
    gf[2] = f2{f20, f21};
    gf[3] = f2{f30, f31};
  }

  // D: GEMM2, dacc += (s (1 - s))^T (g X_aug): features 0 .. 15 as one 16x16 tile per hidden tile,
  // features 16 .. D0 + 1 as 4x4 blocks
  __device__ __forceinline__ void gemm2(const f4 (&dlt)[NT], const float (&ge)[4], const f2 (&gf)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
        dacc_e[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(dlt[t][j], ge[j], dacc_e[t], 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        dacc_f[t][0] = __builtin_amdgcn_mfma_f32_4x4x1f32(dlt[t][j], gf[j][0], dacc_f[t][0], 0, 0, 0);
        dacc_f[t][1] = __builtin_amdgcn_mfma_f32_4x4x1f32(dlt[t][j], gf[j][1], dacc_f[t][1], 0, 0, 0);
      }
    }
  }

  // Software-pipelined loop over full, aligned tiles [tb, te).  Iteration i issues the loads of tile
  // i + 2, GEMM1 of tile i + 1, the pointwise work of tile i and GEMM2 of tile i - 1, all in one
  // basic block.
  template <int LIK, bool LAST>
  __device__ __forceinline__ void fast_loop(const StepCtx& cx, const ModelConsts& mc, int tb, int te,
                                            int n, int q) {
    const PlainPtrs pp = plain_ptrs(cx, tb, n, q);
    TileIn t0, t1, t2;  // tiles i, i + 1, i + 2
    f4 acc_cur[NT], acc_nxt[NT], dlt_prev[NT];
    float ge_prev[4];
    f2 gf_prev[4];
    load_plain(t0, pp, tb);
    load_plain(t1, pp, tb + 1 < te ? tb + 1 : tb);
    gemm1(t0.xa, acc_cur);
#pragma unroll
    for (int t = 0; t < NT; ++t) dlt_prev[t] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      ge_prev[j] = 0.0f;
      gf_prev[j] = f2{0.f, 0.f};
    }
    for (int i = tb; i < te; ++i) {
      load_plain(t2, pp, i + 2 < te ? i + 2 : te - 1);
      gemm1(t1.xa, acc_nxt);                  // tile i + 1
      gemm2(dlt_prev, ge_prev, gf_prev);      // tile i - 1 (zero operands at i = tb)
      float ge[4];
      f2 gf[4];
      pointwise<LIK, LAST, true>(acc_cur, t0, ge, gf, cx, mc, i * 16, n, q);  // tile i
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        dlt_prev[t] = acc_cur[t];
        acc_cur[t] = acc_nxt[t];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        ge_prev[j] = ge[j];
        gf_prev[j] = gf[j];
      }
      t0 = t1;
      t1 = t2;
    }
    gemm2(dlt_prev, ge_prev, gf_prev);  // tile te - 1
  }

  // Plain loop over full, aligned tiles [tb, te): loads two tiles ahead (as far as the compiler
  // leaves them there), then GEMM1, pointwise work and GEMM2 of the current tile back to back.
  template <int LIK, bool LAST>
  __device__ __forceinline__ void simple_loop(const StepCtx& cx, const ModelConsts& mc, int tb,
                                              int te, int n, int q) {
    const PlainPtrs pp = plain_ptrs(cx, tb, n, q);
    TileIn cur, nx1, nx2;
    load_plain(cur, pp, tb);
    load_plain(nx1, pp, tb + 1 < te ? tb + 1 : te - 1);
    for (int i = tb; i < te; ++i) {
      load_plain(nx2, pp, i + 2 < te ? i + 2 : te - 1);
      f4 acc[NT];
      float ge[4];
      f2 gf[4];
      gemm1(cur.xa, acc);
      pointwise<LIK, LAST, true>(acc, cur, ge, gf, cx, mc, i * 16, n, q);
      gemm2(acc, ge, gf);
      cur = nx1;
      nx1 = nx2;
    }
  }

  // ---- explicitly prefetched loop ----
  // The compiler sinks ordinary loads of read-only data next to their first use, which undoes any
  // prefetch written in the source.  Here the loads are issued by inline assembly, which it neither
  // moves nor waits for, two tiles ahead of their use into three rotating register sets, and the
  // waits are explicit: s_waitcnt vmcnt(2 * N_LOADS) leaves the two newer tiles in flight.
  // Memory operations the compiler adds on its own (the last step's log-likelihood rows, spills)
  // only make these waits more conservative, never too short: vmcnt counts every outstanding
  // operation in issue order.
  static constexpr int N_LOADS = 11;
  struct TileRaw {
    f4 xa01;  // GEMM1 operand, k-pairs 0 and 1
    TileIn t; // t.xa[KP - 1]: k-pair 2 (the (1, 0) constant in lane group q = 3); t.xa[0 .. 1] are
              // filled from xa01 when the tile is used
  };
  template <int N>
  static __device__ __forceinline__ void wait_tile(TileRaw& r) {
    asm volatile("s_waitcnt vmcnt(%[cnt])"
                 : "+v"(r.xa01), "+v"(r.t.xa[KP - 1]), "+v"(r.t.xe[0]), "+v"(r.t.xe[1]), "+v"(r.t.xe[2]),
                   "+v"(r.t.xe[3]), "+v"(r.t.xf[0]), "+v"(r.t.xf[1]), "+v"(r.t.xf[2]), "+v"(r.t.xf[3]),
                   "+v"(r.t.y1)
                 : [cnt] "n"(N)
                 : "memory");
  }

  // Every load is  base (wave-uniform, in SGPRs, advanced by scalar instructions)  +  a 32-bit
  // per-lane offset that never changes: no vector instruction is spent on addresses.  Lanes whose
  // operand slot is the constant-one feature or padding do not load at all: their registers are
  // set once (preset) and the loads of those slots run with these lanes masked out of EXEC.
  struct LoadPlan {
    unsigned oa, ol, oe, of, oy;
    unsigned long long mask_a, mask_f;
    int jj;
  };
  static __device__ __forceinline__ LoadPlan load_plan(int n, int q) {
    LoadPlan lp;
    lp.jj = n & 3;
    lp.oa = (unsigned)((n * D0 + KS * q) * 4);
    lp.ol = lp.oa + 2 * (KP - 1) * 4;
    lp.oe = (unsigned)(((4 * q) * D0 + n) * 4);
    lp.of = (unsigned)(((4 * q) * D0 + 16 + 2 * lp.jj) * 4);
    lp.oy = (unsigned)((4 * q + (n >> 2)) * 4);
    const bool a_const = KS * q + 2 * (KP - 1) >= D0;
    const bool f_const = 16 + 2 * lp.jj >= D0;
    lp.mask_a = __builtin_amdgcn_ballot_w64(!a_const);
    lp.mask_f = __builtin_amdgcn_ballot_w64(!f_const);
    return lp;
  }
  static __device__ __forceinline__ void preset(TileRaw& r, int jj) {
    r.t.xa[KP - 1] = f2{1.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < 4; ++j) r.t.xf[j] = const_f(jj);
  }
  // exactly N_LOADS loads of one full tile
  static __device__ __forceinline__ void issue_tile(TileRaw& r, const StepCtx& cx, const LoadPlan& lp, int tile) {
    const float* bx = cx.X + (size_t)tile * (16 * D0);
    const float* by = cx.y + (size_t)tile * 16;
    // One block for the eleven loads.  The leading s_nop gives the five wait states a memory
    // instruction needs after a VALU instruction wrote one of its SGPR operands (the compiler
    // reloads spilled SGPRs with v_readlane and does not see the loads inside the assembly, so it
    // would not insert them itself).  EXEC is saved on entry and put back.  The pure outputs are
    // early-clobber: a returning load must not land in a register that still holds an offset of a
    // load not yet issued.
    unsigned long long exec_save;
    asm volatile(
        "s_mov_b64 %[sv], exec\n\t"
        "s_nop 3\n\t"
        "global_load_dwordx4 %[xa01], %[oa], %[bx]\n\t"
        "global_load_dword %[xe0], %[oe], %[bx]\n\t"
        "global_load_dword %[xe1], %[oe], %[bx] offset:%[r1]\n\t"
        "global_load_dword %[xe2], %[oe], %[bx] offset:%[r2]\n\t"
        "global_load_dword %[xe3], %[oe], %[bx] offset:%[r3]\n\t"
        "global_load_dword %[y1], %[oy], %[by]\n\t"
        "s_and_b64 exec, %[sv], %[ma]\n\t"
        "global_load_dwordx2 %[xa2], %[ol], %[bx]\n\t"
        "s_and_b64 exec, %[sv], %[mf]\n\t"
        "global_load_dwordx2 %[xf0], %[of], %[bx]\n\t"
        "global_load_dwordx2 %[xf1], %[of], %[bx] offset:%[r1]\n\t"
        "global_load_dwordx2 %[xf2], %[of], %[bx] offset:%[r2]\n\t"
        "global_load_dwordx2 %[xf3], %[of], %[bx] offset:%[r3]\n\t"
        "s_mov_b64 exec, %[sv]"
        : [xa01] "=&v"(r.xa01), [xa2] "+v"(r.t.xa[KP - 1]), [xe0] "=&v"(r.t.xe[0]), [xe1] "=&v"(r.t.xe[1]),
          [xe2] "=&v"(r.t.xe[2]), [xe3] "=&v"(r.t.xe[3]), [xf0] "+v"(r.t.xf[0]), [xf1] "+v"(r.t.xf[1]),
          [xf2] "+v"(r.t.xf[2]), [xf3] "+v"(r.t.xf[3]), [y1] "=&v"(r.t.y1), [sv] "=&s"(exec_save)
        : [oa] "v"(lp.oa), [ol] "v"(lp.ol), [oe] "v"(lp.oe), [of] "v"(lp.of), [oy] "v"(lp.oy), [bx] "s"(bx),
          [by] "s"(by), [ma] "s"(lp.mask_a), [mf] "s"(lp.mask_f), [r1] "n"(D0 * 4), [r2] "n"(2 * D0 * 4),
          [r3] "n"(3 * D0 * 4)
        : "memory", "scc");
  }

  // the tiles of the fast loop: full, aligned tiles [tile_begin, fast_end)
  static __device__ __forceinline__ int fast_end_of(const StepCtx& cx) {
    int fast_end = cx.tile_begin;
    if (cx.x_vec_ok && cx.y_vec_ok) fast_end = min(cx.tile_end, cx.n / 16);
    return fast_end;
  }

  // The data does not change from one gradient evaluation to the next, only the weights do: a wave
  // goes round its tiles in a circle, and the loop of one evaluation ends with the first two tiles of
  // the next already in registers (pa, pb), fetched while its own last tiles were being computed, so
  // that no evaluation starts by waiting for memory.  prime() fetches them for the first evaluation.
  TileRaw pa, pb;
  __device__ __forceinline__ void prime(const StepCtx& cx) {
    if (PIPE != 2) return;
    const int tb = cx.tile_begin, te = fast_end_of(cx);
    if (te <= tb) return;
    const int lane = opaque_tid() & 63;
    const LoadPlan lp = load_plan(lane & 15, lane >> 4);
    preset(pa, lp.jj);
    preset(pb, lp.jj);
    issue_tile(pa, cx, lp, tb);
    issue_tile(pb, cx, lp, tb + 1 < te ? tb + 1 : tb);
    wait_tile<0>(pa);
    wait_tile<0>(pb);
  }

  template <int LIK, bool LAST>
  __device__ __forceinline__ void prefetch_loop(const StepCtx& cx, const ModelConsts& mc, int tb,
                                                int te, int n, int q) {
    static_assert(KP == 3, "register sets are laid out for three k-pairs");
    const LoadPlan lp = load_plan(n, q);
    // tiles are issued in order, one call each, and after the last tile comes the first again; on
    // entry pa and pb hold tiles tb and tb + 1 (tb again if there is only one)
    int nxt = te - tb > 2 ? tb + 2 : tb;
    auto issue = [&](TileRaw& r) {
      issue_tile(r, cx, lp, nxt);
      nxt = nxt + 1 == te ? tb : nxt + 1;
    };
    auto compute = [&](TileRaw& r, int tile) {
      r.t.xa[0] = f2{r.xa01[0], r.xa01[1]};
      r.t.xa[1] = f2{r.xa01[2], r.xa01[3]};
      f4 acc[NT];
      float ge[4];
      f2 gf[4];
      gemm1(r.t.xa, acc);
      pointwise<LIK, LAST, true>(acc, r.t, ge, gf, cx, mc, tile * 16, n, q);
      // keep the stages apart: left to itself the scheduler may feed each GEMM2 operand to its
      // MFMAs the moment it is computed, which puts two wait states in front of every other MFMA
      __builtin_amdgcn_sched_barrier(0);
      gemm2(acc, ge, gf);
      __builtin_amdgcn_sched_barrier(0);
    };
    TileRaw& A = pa;
    TileRaw& B = pb;
    TileRaw C;
    preset(C, lp.jj);
    // steady state: three tiles per trip, every issue and every wait unconditional.
    // Two waves share a SIMD, and the matrix and vector instructions of both go through one FP32
    // pipe: it stays busy only while both waves have work (each fills the dependency stalls of the
    // other).  The hardware favours the older wave, which would finish its tiles long before the
    // younger one and leave it to run alone, stalls exposed.  So every trip a wave publishes its
    // tile count in LDS, reads its partner's, and takes the higher priority while it is behind
    // (once per trip of three tiles: checked after every tile the kernel was 3 % slower).
    int i = tb;
    const bool balance = cx.progress != nullptr;
    auto keep_pace = [&](int done) {
      if (balance) {
        // all operands are wave-uniform: the registers live only across these three instructions
        const unsigned my_slot = (unsigned)(size_t)(cx.progress + cx.wave);  // LDS byte addresses
        const unsigned other_slot = (unsigned)(size_t)(cx.progress + cx.partner);
        int other;
        asm volatile("ds_write_b32 %1, %2\n\tds_read_b32 %0, %3\n\ts_waitcnt lgkmcnt(0)"
                     : "=&v"(other)
                     : "v"(my_slot), "v"(done), "v"(other_slot)
                     : "memory");
        if (__builtin_amdgcn_readfirstlane(other) > done) __builtin_amdgcn_s_setprio(2);
        else __builtin_amdgcn_s_setprio(0);
      }
    };
    for (; i + 3 <= te; i += 3) {
      issue(C);
      wait_tile<2 * N_LOADS>(A);
      compute(A, i);
      issue(A);
      wait_tile<2 * N_LOADS>(B);
      compute(B, i + 1);
      issue(B);
      wait_tile<2 * N_LOADS>(C);
      compute(C, i + 2);
      keep_pace(i + 3 - tb);
    }
    if (balance) __builtin_amdgcn_s_setprio(0);
    // the one or two tiles left over sit in A and B (issued at the end of the last trip); the
    // loads issued from here on are the first tiles of the next evaluation
    const int left = te - i;
    if (left >= 1) {
      issue(C);
      wait_tile<2 * N_LOADS>(A);
      compute(A, i);
    }
    if (left == 2) {
      issue(A);
      wait_tile<2 * N_LOADS>(B);
      compute(B, i + 1);
    }
    // no register of a set may be used or reused before its last load has landed
    wait_tile<0>(A);
    wait_tile<0>(B);
    wait_tile<0>(C);
    // tiles tb and tb + 1 back into (pa, pb)
    if (left == 1) {
      A = B;
      B = C;
    } else if (left == 2) {
      const TileRaw first = C;
      B = A;
      A = first;
    }
  }

  template <int LIK, bool LAST>
  __device__ __forceinline__ void run_tiles(const StepCtx& cx, const ModelConsts& mc) {
    const int lane = opaque_tid() & 63, n = lane & 15, q = lane >> 4;
    const int tb = cx.tile_begin, te = cx.tile_end;
    const int fast_end = fast_end_of(cx);
    if (fast_end > tb) {
      if (PIPE == 1) fast_loop<LIK, LAST>(cx, mc, tb, fast_end, n, q);
      else if (PIPE == 2) prefetch_loop<LIK, LAST>(cx, mc, tb, fast_end, n, q);
      else simple_loop<LIK, LAST>(cx, mc, tb, fast_end, n, q);
    }
    // ragged tail tile, or unaligned caller buffers: one tile at a time
    for (int tile = max(tb, fast_end); tile < te; ++tile) {
      TileIn ti;
      f4 acc[NT];
      float ge[4];
      f2 gf[4];
      load_tile_safe(ti, cx, tile * 16, n, q);
      gemm1(ti.xa, acc);
      pointwise<LIK, LAST, false>(acc, ti, ge, gf, cx, mc, tile * 16, n, q);
      gemm2(acc, ge, gf);
    }
  }

  // a (lower half) + a (upper half) in lanes 0 .. 31 and the same of b in lanes 32 .. 63; one lane
  // swap and one addition, no trip through LDS.  Written in assembly because the compiler's builtin
  // for the swap hands back its two results in one register at -O3.  The s_nop is the two wait states
  // the swap needs after a vector instruction wrote one of its operands; the operands must come from
  // ordinary vector instructions (not straight from an MFMA, whose longer hazard the compiler cannot
  // see through the assembly).
  static __device__ __forceinline__ float fold32(float a, float b) {
    asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    return a + b;
  }
  // rows of 16 lanes: (a row 0 + a row 1, b row 0 + b row 1, a row 2 + a row 3, b row 2 + b row 3)
  static __device__ __forceinline__ float fold16(float a, float b) {
    asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    return a + b;
  }

  // ---- the wave's partial sums in LDS ----
  // A wave's slot is a table of 48-float rows: row f < D0 holds the sums for feature f, row D0 those of
  // the bias, row 24 those of the layer-2 weights, row 25 the log-likelihood difference; column c is
  // the hidden unit (columns D1 .. 47 are the padded units: the first of them, in the bias row, holds the
  // sum for b2).  With rows of 48 every lane stores whole registers unconditionally.
  static constexpr int ROW = 16 * NT;
  static constexpr int W2_ROW = 24, DL_ROW = 25;
  static constexpr int LDS_SLOT = (DL_ROW + 1) * ROW;
  static constexpr int DL_INDEX = DL_ROW * ROW;
  static __device__ __forceinline__ int slot_index(int p) {
    if (p < oW2) return (p / D1) * ROW + p % D1;  // W1 rows, then the bias row (oB1 = D0 D1)
    if (p < oB2) return W2_ROW * ROW + (p - oW2);
    return D0 * ROW + D1;
  }
  // What a sum over the waves' slots still lacks: the factors 4 w2[c] left out of the GEMM2 operand and
  // k / k2 left out of g (applied once per workgroup, after the sum, not once per wave).
  template <int LIK>
  __device__ __forceinline__ float finish(int p, float v, const float* s_w) const {
    const float gr = LIK == 1 ? ratio : 1.0f;
    if (p < oW2) return v * (4.0f * gr * s_w[oW2 + p % D1]);
    if (p < oB2) return v * gr;
    return v * (4.0f * gr);
  }

  // this wave's partial sums -> its LDS slot (layout above).  `last`: the log-likelihood difference of
  // the step is written too.
  template <int LIK>
  __device__ __forceinline__ void write_partials(float* slot, const float*, bool last) {
    const int lane = opaque_tid() & 63, n = lane & 15, q = lane >> 4;
    static_assert(D1 % 16 != 0, "db2 rides in the first padded hidden unit");
    static_assert(NT == 3, "the row-group sums below are laid out for three hidden tiles");
    static_assert(D0 + 2 <= W2_ROW, "feature rows end below the layer-2 row");
    // The accumulators of features 16 .. D0 + 1 and of dw2 hold one partial per row group q (the four
    // rows of 16 lanes); two folds add the four partials of four registers at once and leave each row
    // of lanes with the total of one of them.  After
    //     fold16(fold32(x0, y0), fold32(x1, y1))
    // row q holds the total of (q & 1 ? x1 : x0) for q < 2 and of (q & 1 ? y1 : y0) for q >= 2,
    // added as (q0 + q2) + (q1 + q3).
    // ---- features 0 .. 15: lane (n, q), component i: c = 16 t + 4 q + i, f = n ----
#pragma unroll
    for (int t = 0; t < NT; ++t)
      *reinterpret_cast<f4*>(slot + n * ROW + 16 * t + 4 * q) = dacc_e[t];
    // ---- features 16 .. D0 + 1: before the folds lane (n, q), component i holds
    //      c = 16 t + 4 (n >> 2) + i, f = 16 + 2 (n & 3) + fb for row group q; after them the lane
    //      holds c = 16 t + cb + 2 h and f = 16 + 2 (n & 3) + (q >> 1).  f = D0 is the bias; the sum of g
    //      over the wave's rows (db2) has gathered in the first padded hidden unit ----
    const int cb = 4 * (n >> 2) + (q & 1);
    const int f = 16 + 2 * (n & 3) + (q >> 1);
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const float v = fold16(fold32(dacc_f[t][0][2 * h], dacc_f[t][1][2 * h]),
                               fold32(dacc_f[t][0][2 * h + 1], dacc_f[t][1][2 * h + 1]));
        slot[f * ROW + 16 * t + cb + 2 * h] = v;
      }
    }
    // ---- dw2 = sum_rows g h = 2 (sum_rows g s - sum_rows g / 2); the second sum is what the first
    //      padded hidden unit (lane n = D1 % 16 of the last hidden tile, s = 1/2) has accumulated ----
    {
      const float half_gsum = dpp_move<0x150 + D1 % 16>(dw2s[NT - 1]);  // row_newbcast
      const float v0 = 2.0f * (dw2s[0] - half_gsum);
      const float v1 = 2.0f * (dw2s[1] - half_gsum);
      const float v2 = 2.0f * (dw2s[2] - half_gsum);
      const float v = fold16(fold32(v0, v1), fold32(v2, v2));  // rows: tile 0, tile 2, tile 1, tile 2
      const int t = q == 0 ? 0 : (q == 2 ? 1 : 2);
      slot[W2_ROW * ROW + 16 * t + n] = v;  // (rows 1 and 3 store the same bits to the same place)
    }
    if (last) {
      double d = dl;  // held by lanes n == 0
      d += shfl_xor_d(d, 16);
      d += shfl_xor_d(d, 32);
      if (lane == 0) {
        const uint64_t bits = double_to_bits(d);
        slot[DL_INDEX] = __builtin_bit_cast(float, (uint32_t)bits);
        slot[DL_INDEX + 1] = __builtin_bit_cast(float, (uint32_t)(bits >> 32));
      }
    }
  }
};

}  // namespace bnn
