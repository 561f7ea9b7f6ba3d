// The MFMA layer of the 22 -> 40 -> 1 trajectory kernel with no padded hidden units: hidden units 0 .. 31
// go through two 16-wide tiles of v_mfma_f32_16x16x4_f32 as in MfmaLayer (bnn_mfma_layer.h); hidden units
// 32 .. 39, which there occupy a third tile that is half empty, go through v_mfma_f32_4x4x1_16b_f32 (sixteen
// independent 4x4 blocks per instruction) in both contractions, and the pointwise stage runs on the 40 real
// hidden units only (10 values per lane instead of 12).  Per 16-row tile: 20 wide + 40 block matrix
// instructions instead of 30 + 24, 20 transcendentals instead of 24.
//
// The block instructions want their operands per block -- rows and features of x in layouts that differ from
// the ones the wide instructions read -- so a wave keeps a copy of the current tile in LDS (16 rows x 24
// floats, written from the registers of the GEMM1 operand, which hold every element of the tile exactly
// once) and reads from it what the block instructions and the 4x4 part of GEMM2 need.  What is prefetched
// from memory into registers is therefore only the GEMM1 operand, the GEMM2 operand of features 0 .. 15 and
// the targets (7 loads and 11 registers per tile instead of 11 and 23).
//
// Lane l = 16 q + n, n = 4 cb + r, h8 = n >> 3, c8 = n & 7.
//   GEMM1, hidden 32 .. 39: twelve block instructions s = 0 .. 11, block b = 4 q + cb:
//        A_b[i] = x_aug[row 4 q + i][k = 12 (cb >> 1) + s]       (lane 4 cb + i supplies it: x5a[s])
//        B_b[r] = k W1_aug[k][32 + 4 (cb & 1) + r]                (lane 4 cb + r: w5[s])
//        D: lane (n, q), register i: row 4 q + i, hidden 32 + c8, partial over the k-half h8
//      folded (4 bank-masked DPP additions) so that lanes n < 8 hold the totals of rows 4 q, 4 q + 1 and
//      lanes n >= 8 those of rows 4 q + 2, 4 q + 3: two values per lane (sa, sb), rows ra = 4 q + 2 h8, ra + 1.
//   GEMM2: g rides on the A operand (u g), the rows of x are used as loaded.
//        hidden 0 .. 31, features 0 .. 15: wide instructions, as MfmaLayer
//        hidden 0 .. 31, features 16 .. 23: block instructions, as MfmaLayer (operand from the LDS copy)
//        hidden 32 .. 39: twelve block instructions (rho = 0, 1; fs = 0 .. 5):
//            A_b[i] = u g of hidden 32 + 4 (cb & 1) + i, row ra + rho     (lane 4 cb + i: uga / ugb)
//            B_b[r] = x_aug[row ra + rho][feature 6 r + fs]                (lane 4 cb + r: from the LDS copy)
//            D: lane (n, q), register i of d5[fs]: hidden 32 + 4 (cb & 1) + i, feature 6 r + fs,
//               partial over the rows {ra, ra + 1} of all tiles
#pragma once

#include <hip/hip_runtime.h>

#include "bnn_device.h"
#include "bnn_kernel_common.h"
#include "bnn_mfma_layer.h"

namespace bnn {

template <int D0, int D1>
struct MfmaHybridLayer {
  static_assert(D0 == 22 && D1 == 40, "laid out for 22 features (24 with the bias and one pad) and 32 + 8 hidden units");
  static constexpr int KS = 6, KP = 3;  // k-steps of the wide GEMM1: 24 = 4 x 6
  static constexpr int NT = 2;          // 16-wide hidden tiles
  static constexpr int oB1 = D0 * D1, oW2 = oB1 + D1, oB2 = oW2 + D1, P = oB2 + 1;
  static constexpr int P_AL = (P + 3) / 4 * 4;
  static constexpr int TILE_LDS = 16 * 24;  // floats of a wave's copy of the current tile
  static constexpr float kExp2Scale = -2.88539008177792681472f;  // -2 / ln 2, kernel_helpers.h:37

  // per step (see MfmaLayer for the meaning of the scalings)
  float w1b[KS][NT];   // hidden 0 .. 31: k W1_aug[6 q + s][16 t + n]
  float w5[12];        // hidden 32 .. 39: k W1_aug[12 h8 + s][32 + c8]
  float w2g[NT], w2g5; // -2 w2[c] k2
  float k2v, y_0, rho, ratio;
  // sums over rows
  f4 dacc_e[NT];       // hidden 16 t + 4 q + i, feature n
  f4 dacc_f[NT][2];    // hidden 16 t + 4 cb + i, feature 16 + 2 r + fb, partial over row group q
  f4 d5[6];            // see above
  float dw2s[NT];      // sum over the rows of group q of g' s, hidden 16 t + n
  float dw2s5;         // sum over the rows ra, ra + 1 of g' (s - 1/2), hidden 32 + c8
  float hs;            // sum over the rows of group q of g' / 2, added in the very order of dw2s: dw2 =
                       // 2 (dw2s - hs) is exactly zero where every s is 1/2 (all weights zero)
  double dl;

  struct TileIn {
    f2 xa[KP];   // GEMM1 operand: row n, k = 6 q + 2 i, + 1
    float y1;    // target of row 4 q + (n >> 2)
  };

  template <int LIK>
  __device__ __forceinline__ void load_weights(const float* s_w, const ModelConsts& mc) {
    const int lane = opaque_tid() & 63, n = lane & 15, q = lane >> 4, h8 = n >> 3, c8 = n & 7;
    const float k = LIK == 1 ? mc.scale_recp * mc.scale_recp : mc.scale_recp;
    const uint32_t k2_bits = (__builtin_bit_cast(uint32_t, k) + 0x00400000u) & 0x7F800000u;
    const float k2 = __builtin_bit_cast(float, k2_bits);
    ratio = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(
        int, k * __builtin_bit_cast(float, 0x7F000000u - k2_bits))));
    double w2lane = 0.0;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int c = 16 * t + n;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const int kk = KS * q + s;
        const float v = s_w[kk < D0 ? kk * D1 + c : oB1 + c];  // kk == D0: the bias row; beyond: padding
        w1b[s][t] = kk <= D0 ? v * kExp2Scale : 0.0f;
      }
      const float w2c = s_w[oW2 + c];
      w2lane += (double)w2c;
      w2g[t] = -2.0f * w2c * k2;
    }
    {
      const int c = 32 + c8;
#pragma unroll
      for (int s = 0; s < 12; ++s) {
        const int kk = 12 * h8 + s;
        const float v = s_w[kk < D0 ? kk * D1 + c : oB1 + c];
        w5[s] = kk <= D0 ? v * kExp2Scale : 0.0f;
      }
      const float w2c = s_w[oW2 + c];
      // a lane's share of the constant covers hidden 32 + n once (lanes n < 8)
      if (h8 == 0) w2lane += (double)w2c;
      w2g5 = -2.0f * w2c * k2;
    }
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
#pragma unroll
    for (int fs = 0; fs < 6; ++fs) d5[fs] = f4{0.f, 0.f, 0.f, 0.f};
    dw2s5 = 0.0f;
    hs = 0.0f;
    dl = 0.0;
  }

  // rows past the end read as the last row (their gradient is masked to zero); any alignment
  __device__ __forceinline__ void load_tile_safe(TileIn& ti, const StepCtx& cx, int row0, int n, int q) const {
    const int last = cx.n - 1;
    const float* ra = cx.X + (size_t)min(row0 + n, last) * D0;
#pragma unroll
    for (int i = 0; i < KP; ++i) {
      const int k0 = KS * q + 2 * i;
      const int kc = k0 < D0 ? k0 : D0 - 2;
      f2 v = f2{ra[kc], ra[kc + 1]};
      if (k0 >= D0) v = f2{k0 == D0 ? 1.0f : 0.0f, 0.0f};
      ti.xa[i] = v;
    }
    ti.y1 = cx.y[min(row0 + 4 * q + (n >> 2), last)];
  }

  static __device__ __forceinline__ f4 mfma4(float a, float b, f4 c) {
    return __builtin_amdgcn_mfma_f32_4x4x1f32(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f4 mfma16(float a, float b, f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
  }

  // One tile: the LDS copy, GEMM1, the pointwise stage, GEMM2.  `tile` is this wave's LDS buffer.
  template <int LIK, bool LAST, bool FULL>
  __device__ __forceinline__ void compute_tile(const TileIn& ti, float* tile, const StepCtx& cx,
                                               const ModelConsts& mc, int row0, int n, int q) {
    const int r = n & 3, h8 = n >> 3;
    const int ra = 4 * q + 2 * h8;
    // ---- the wave's copy of the tile: lane (n, q) holds x_aug[row n][6 q .. 6 q + 5] ----
    {
      f2* dst = reinterpret_cast<f2*>(tile + n * 24 + KS * q);
      dst[0] = ti.xa[0];
      dst[1] = ti.xa[1];
      dst[2] = ti.xa[2];
    }
    // GEMM1 operand of the block instructions: x_aug[row 4 q + r][12 h8 .. 12 h8 + 11]
    f4 x5a[3];
    {
      const f4* src = reinterpret_cast<const f4*>(tile + (4 * q + r) * 24 + 12 * h8);
      x5a[0] = src[0];
      x5a[1] = src[1];
      x5a[2] = src[2];
    }
    // ---- GEMM1 ----
    f4 acc[NT] = {f4{0.f, 0.f, 0.f, 0.f}, f4{0.f, 0.f, 0.f, 0.f}};
    f4 acc5 = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < KP; ++i) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        acc[0] = mfma16(ti.xa[i][h], w1b[2 * i + h][0], acc[0]);
        acc[1] = mfma16(ti.xa[i][h], w1b[2 * i + h][1], acc[1]);
      }
    }
#pragma unroll
    for (int s = 0; s < 12; ++s) acc5 = mfma4(x5a[s >> 2][s & 3], w5[s], acc5);
    // the GEMM2 operands that come from the LDS copy: issued here, used after the pointwise stage
    float xe[4];   // x[row 4 q + j][n]
    f2 xf[4];      // x_aug[row 4 q + j][16 + 2 r, 17 + 2 r]
    f2 x5b[2][3];  // x_aug[row ra + rho][6 r .. 6 r + 5]
#pragma unroll
    for (int j = 0; j < 4; ++j) xe[j] = tile[(4 * q + j) * 24 + n];
#pragma unroll
    for (int j = 0; j < 4; ++j) xf[j] = *reinterpret_cast<const f2*>(tile + (4 * q + j) * 24 + 16 + 2 * r);
#pragma unroll
    for (int rh = 0; rh < 2; ++rh) {
      const f2* src = reinterpret_cast<const f2*>(tile + (ra + rh) * 24 + 6 * r);
      x5b[rh][0] = src[0];
      x5b[rh][1] = src[1];
      x5b[rh][2] = src[2];
    }
    __builtin_amdgcn_sched_barrier(0);
    // ---- the two k-halves of hidden 32 .. 39: lanes n < 8 keep rows 4 q, 4 q + 1 (registers 0, 1), lanes
    //      n >= 8 rows 4 q + 2, 4 q + 3 (registers 2, 3).  The leading s_nop covers the wait states a vector
    //      instruction needs after a block matrix instruction wrote its operand (the compiler does not see
    //      the reads inside the assembly) ----
    float sa = acc5[2], sb = acc5[3];
    asm volatile("s_nop 7\n\t"
                 "v_add_f32_dpp %[a], %[a], %[a] row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                 "v_add_f32_dpp %[b], %[b], %[b] row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                 "v_add_f32_dpp %[a], %[p0], %[p0] row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
                 "v_add_f32_dpp %[b], %[p1], %[p1] row_ror:8 row_mask:0xf bank_mask:0x3"
                 : [a] "+v"(sa), [b] "+v"(sb)
                 : [p0] "v"(acc5[0]), [p1] "v"(acc5[1]));
    // ---- pointwise stage (logistic form, see MfmaLayer::pointwise) ----
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
    sa = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(sa));
    sb = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(sb));
    // hidden 32 .. 39 in the row sums: a lane holds two of its four rows
    asm("s_nop 1\n\t"
        "v_fmac_f32_dpp %[y0], %[a], %[w] quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0x3\n\t"
        "v_fmac_f32_dpp %[y2], %[a], %[w] quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0xc\n\t"
        "v_fmac_f32_dpp %[y1], %[b], %[w] quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0x3\n\t"
        "v_fmac_f32_dpp %[y3], %[b], %[w] quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0xc"
        : [y0] "+v"(yh[0]), [y1] "+v"(yh[1]), [y2] "+v"(yh[2]), [y3] "+v"(yh[3])
        : [a] "v"(sa), [b] "v"(sb), [w] "v"(w2g5));
    // (y - yhat - b2) k2 of the four rows 4 q + j, in bank j of one register
    const float rz = row16_reduce4(yh[0], yh[1], yh[2], yh[3]) + __builtin_fmaf(ti.y1, k2v, rho);
    float gz = rz, dz = rz;
    if (LIK == 0) {
      dz = rz * ratio;
      gz = dz * mc.g_scale * __builtin_amdgcn_rcpf(__builtin_fmaf(dz, dz, mc.df));
    }
    if (!FULL) gz = row0 + 4 * q + (n >> 2) < cx.n ? gz : 0.0f;  // mcmc_step_ffma.h:301 (the lane's bank holds that row)
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
    // dw2s += g s, hs += g / 2 (same order), dw2s5 += g (s - 1/2); then u g = (s - s^2) g in place.  g of row
    // 4 q + j is read from bank j of gz through a DPP row broadcast; for hidden 32 .. 39 lanes n < 8 take the
    // rows 4 q, 4 q + 1 (banks 0, 1) and lanes n >= 8 the rows 4 q + 2, 4 q + 3 (banks 2, 3).
    const float sa_c = sa - 0.5f, sb_c = sb - 0.5f;
    float uga = __builtin_fmaf(-sa, sa, sa), ugb = __builtin_fmaf(-sb, sb, sb);
    const float half = 0.5f;
#define BNN_BC(j) " row_newbcast:" #j " row_mask:0xf bank_mask:0xf\n\t"
    asm("s_nop 1\n\t"
        "v_fmac_f32_dpp %[d0], %[g], %[s00]" BNN_BC(0)
        "v_fmac_f32_dpp %[d1], %[g], %[s10]" BNN_BC(0)
        "v_fmac_f32_dpp %[hs], %[g], %[hf]" BNN_BC(0)
        "v_fmac_f32_dpp %[d0], %[g], %[s01]" BNN_BC(4)
        "v_fmac_f32_dpp %[d1], %[g], %[s11]" BNN_BC(4)
        "v_fmac_f32_dpp %[hs], %[g], %[hf]" BNN_BC(4)
        "v_fmac_f32_dpp %[d0], %[g], %[s02]" BNN_BC(8)
        "v_fmac_f32_dpp %[d1], %[g], %[s12]" BNN_BC(8)
        "v_fmac_f32_dpp %[hs], %[g], %[hf]" BNN_BC(8)
        "v_fmac_f32_dpp %[d0], %[g], %[s03]" BNN_BC(12)
        "v_fmac_f32_dpp %[d1], %[g], %[s13]" BNN_BC(12)
        "v_fmac_f32_dpp %[hs], %[g], %[hf]" BNN_BC(12)
        "v_fmac_f32_dpp %[d5], %[g], %[sa] row_newbcast:0 row_mask:0xf bank_mask:0x3\n\t"
        "v_fmac_f32_dpp %[d5], %[g], %[sa] row_newbcast:8 row_mask:0xf bank_mask:0xc\n\t"
        "v_fmac_f32_dpp %[d5], %[g], %[sb] row_newbcast:4 row_mask:0xf bank_mask:0x3\n\t"
        "v_fmac_f32_dpp %[d5], %[g], %[sb] row_newbcast:12 row_mask:0xf bank_mask:0xc"
        : [d0] "+v"(dw2s[0]), [d1] "+v"(dw2s[1]), [hs] "+v"(hs), [d5] "+v"(dw2s5)
        : [g] "v"(gz), [hf] "v"(half), [s00] "v"(acc[0][0]), [s01] "v"(acc[0][1]), [s02] "v"(acc[0][2]),
          [s03] "v"(acc[0][3]), [s10] "v"(acc[1][0]), [s11] "v"(acc[1][1]), [s12] "v"(acc[1][2]),
          [s13] "v"(acc[1][3]), [sa] "v"(sa_c), [sb] "v"(sb_c));
    float ug[NT][4];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma unroll
      for (int j = 0; j < 4; ++j) ug[t][j] = __builtin_fmaf(-acc[t][j], acc[t][j], acc[t][j]);
    }
    asm("s_nop 1\n\t"
        "v_mul_f32_dpp %[u00], %[g], %[u00]" BNN_BC(0)
        "v_mul_f32_dpp %[u10], %[g], %[u10]" BNN_BC(0)
        "v_mul_f32_dpp %[u01], %[g], %[u01]" BNN_BC(4)
        "v_mul_f32_dpp %[u11], %[g], %[u11]" BNN_BC(4)
        "v_mul_f32_dpp %[u02], %[g], %[u02]" BNN_BC(8)
        "v_mul_f32_dpp %[u12], %[g], %[u12]" BNN_BC(8)
        "v_mul_f32_dpp %[u03], %[g], %[u03]" BNN_BC(12)
        "v_mul_f32_dpp %[u13], %[g], %[u13]" BNN_BC(12)
        "v_mul_f32_dpp %[ua], %[g], %[ua] row_newbcast:0 row_mask:0xf bank_mask:0x3\n\t"
        "v_mul_f32_dpp %[ua], %[g], %[ua] row_newbcast:8 row_mask:0xf bank_mask:0xc\n\t"
        "v_mul_f32_dpp %[ub], %[g], %[ub] row_newbcast:4 row_mask:0xf bank_mask:0x3\n\t"
        "v_mul_f32_dpp %[ub], %[g], %[ub] row_newbcast:12 row_mask:0xf bank_mask:0xc"
        : [u00] "+v"(ug[0][0]), [u01] "+v"(ug[0][1]), [u02] "+v"(ug[0][2]), [u03] "+v"(ug[0][3]),
          [u10] "+v"(ug[1][0]), [u11] "+v"(ug[1][1]), [u12] "+v"(ug[1][2]), [u13] "+v"(ug[1][3]),
          [ua] "+v"(uga), [ub] "+v"(ugb)
        : [g] "v"(gz));
#undef BNN_BC
    __builtin_amdgcn_sched_barrier(0);
    // ---- GEMM2 ----
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      dacc_e[0] = mfma16(ug[0][j], xe[j], dacc_e[0]);
      dacc_e[1] = mfma16(ug[1][j], xe[j], dacc_e[1]);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        dacc_f[t][0] = mfma4(ug[t][j], xf[j][0], dacc_f[t][0]);
        dacc_f[t][1] = mfma4(ug[t][j], xf[j][1], dacc_f[t][1]);
      }
    }
#pragma unroll
    for (int fs = 0; fs < 6; ++fs) d5[fs] = mfma4(uga, x5b[0][fs >> 1][fs & 1], d5[fs]);
#pragma unroll
    for (int fs = 0; fs < 6; ++fs) d5[fs] = mfma4(ugb, x5b[1][fs >> 1][fs & 1], d5[fs]);
    __builtin_amdgcn_sched_barrier(0);
  }

  // ---- explicitly prefetched loop (see MfmaLayer::prefetch_loop): loads issued from inline assembly two tiles
  //      ahead into three rotating register sets, explicit waits ----
  static constexpr int N_LOADS = 3;
  struct TileRaw {
    f4 xa01;   // GEMM1 operand, k-pairs 0 and 1
    TileIn t;  // t.xa[2]: k-pair 2 (the (1, 0) constant in lane group q = 3); t.xa[0 .. 1] from xa01 at use
  };
  template <int N>
  static __device__ __forceinline__ void wait_tile(TileRaw& r) {
    asm volatile("s_waitcnt vmcnt(%[cnt])"
                 : "+v"(r.xa01), "+v"(r.t.xa[KP - 1]), "+v"(r.t.y1)
                 : [cnt] "n"(N)
                 : "memory");
  }
  struct LoadPlan {
    unsigned oa, ol, oy;
    unsigned long long mask_a;
  };
  static __device__ __forceinline__ LoadPlan load_plan(int n, int q) {
    LoadPlan lp;
    lp.oa = (unsigned)((n * D0 + KS * q) * 4);
    lp.ol = lp.oa + 2 * (KP - 1) * 4;
    lp.oy = (unsigned)((4 * q + (n >> 2)) * 4);
    const bool a_const = KS * q + 2 * (KP - 1) >= D0;
    lp.mask_a = __builtin_amdgcn_ballot_w64(!a_const);
    return lp;
  }
  static __device__ __forceinline__ void preset(TileRaw& r) { r.t.xa[KP - 1] = f2{1.0f, 0.0f}; }
  // exactly N_LOADS loads of one full tile (see MfmaLayer::issue_tile for the s_nop, EXEC and early-clobber)
  static __device__ __forceinline__ void issue_tile(TileRaw& r, const StepCtx& cx, const LoadPlan& lp, int tile) {
    const float* bx = cx.X + (size_t)tile * (16 * D0);
    const float* by = cx.y + (size_t)tile * 16;
    unsigned long long exec_save;
    asm volatile(
        "s_mov_b64 %[sv], exec\n\t"
        "s_nop 3\n\t"
        "global_load_dwordx4 %[xa01], %[oa], %[bx]\n\t"
        "global_load_dword %[y1], %[oy], %[by]\n\t"
        "s_and_b64 exec, %[sv], %[ma]\n\t"
        "global_load_dwordx2 %[xa2], %[ol], %[bx]\n\t"
        "s_mov_b64 exec, %[sv]"
        : [xa01] "=&v"(r.xa01), [xa2] "+v"(r.t.xa[KP - 1]), [y1] "=&v"(r.t.y1), [sv] "=&s"(exec_save)
        : [oa] "v"(lp.oa), [ol] "v"(lp.ol), [oy] "v"(lp.oy), [bx] "s"(bx), [by] "s"(by), [ma] "s"(lp.mask_a)
        : "memory", "scc");
  }

  static __device__ __forceinline__ int fast_end_of(const StepCtx& cx) {
    int fast_end = cx.tile_begin;
    if (cx.x_vec_ok && cx.y_vec_ok) fast_end = min(cx.tile_end, cx.n / 16);
    return fast_end;
  }

  // A wave walks its run of tiles forwards in one gradient evaluation and backwards in the next (cx.back,
  // cx.back_next): what it read last -- what the caches most likely still hold when the rows of all chains in
  // flight exceed them -- is what it reads first.  The partial sums of a backward evaluation are added in the
  // opposite order, so the direction is a function of the leapfrog step alone, and the last step of a trajectory,
  // whose gradient a chain carries into its next transition (and a resumed chain computes afresh), always goes
  // forwards.
  TileRaw pa, pb;  // the first two tiles of the next evaluation (see MfmaLayer)
  // tile number k of an evaluation's walk over [tb, te)
  static __device__ __forceinline__ int walk(int tb, int te, int k, int back) { return back ? te - 1 - k : tb + k; }
  __device__ __forceinline__ void prime(const StepCtx& cx) {
    const int tb = cx.tile_begin, te = fast_end_of(cx);
    if (te <= tb) return;
    const int lane = opaque_tid() & 63;
    const LoadPlan lp = load_plan(lane & 15, lane >> 4);
    const int back = __builtin_amdgcn_readfirstlane(cx.back);
    preset(pa);
    preset(pb);
    issue_tile(pa, cx, lp, __builtin_amdgcn_readfirstlane(walk(tb, te, 0, back)));
    issue_tile(pb, cx, lp, __builtin_amdgcn_readfirstlane(walk(tb, te, tb + 1 < te ? 1 : 0, back)));
    wait_tile<0>(pa);
    wait_tile<0>(pb);
  }

  template <int LIK, bool LAST>
  __device__ __forceinline__ void prefetch_loop(const StepCtx& cx, const ModelConsts& mc, int tb, int te, int n,
                                                int q) {
    const LoadPlan lp = load_plan(n, q);
    float* tile = cx.tile_lds;
    // the loads run two tiles ahead of the arithmetic along the walk, into the next evaluation's (which goes
    // the other way) at the end of this one's
    const int back = __builtin_amdgcn_readfirstlane(cx.back);
    const int back_next = __builtin_amdgcn_readfirstlane(cx.back_next);
    const int len = te - tb;
    int nk = 2, nback = back;
    while (nk >= len) {  // (a run of one tile is the same tile in either direction)
      nk -= len;
      nback = back_next;
    }
    auto issue = [&](TileRaw& r) {
      issue_tile(r, cx, lp, __builtin_amdgcn_readfirstlane(walk(tb, te, nk, nback)));
      if (++nk == len) {
        nk = 0;
        nback = back_next;
      }
    };
    auto compute = [&](TileRaw& r, int i) {  // i: tb + position in the walk
      r.t.xa[0] = f2{r.xa01[0], r.xa01[1]};
      r.t.xa[1] = f2{r.xa01[2], r.xa01[3]};
      compute_tile<LIK, LAST, true>(r.t, tile, cx, mc, walk(tb, te, i - tb, back) * 16, n, q);
    };
    TileRaw& A = pa;
    TileRaw& B = pb;
    TileRaw C;
    preset(C);
    int i = tb;
    const bool balance = cx.progress != nullptr;
    auto keep_pace = [&](int done) {
      if (balance) {
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
    wait_tile<0>(A);
    wait_tile<0>(B);
    wait_tile<0>(C);
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
    if (fast_end > tb) prefetch_loop<LIK, LAST>(cx, mc, tb, fast_end, n, q);
    // ragged tail tile, or unaligned caller buffers: one tile at a time
    for (int tile = max(tb, fast_end); tile < te; ++tile) {
      TileIn ti;
      load_tile_safe(ti, cx, tile * 16, n, q);
      compute_tile<LIK, LAST, false>(ti, cx.tile_lds, cx, mc, tile * 16, n, q);
    }
  }

  static __device__ __forceinline__ float fold32(float a, float b) {
    asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    return a + b;
  }
  static __device__ __forceinline__ float fold16(float a, float b) {
    asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    return a + b;
  }
  // after fold4(x0, y0, x1, y1) row q of lanes holds the sum over the four rows of lanes of x0 (q = 0),
  // x1 (q = 1), y0 (q = 2), y1 (q = 3), added as (q0 + q2) + (q1 + q3)
  static __device__ __forceinline__ float fold4(float x0, float y0, float x1, float y1) {
    return fold16(fold32(x0, y0), fold32(x1, y1));
  }

  // ---- the wave's partial sums in LDS: the table of MfmaLayer (48-float rows: row f < D0 feature f, row D0
  //      the bias, row 24 the layer-2 weights, row 25 the log-likelihood difference; column = hidden unit,
  //      column D1 of the bias row holds the sum for b2) ----
  static constexpr int ROW = 48;
  static constexpr int W2_ROW = 24, DL_ROW = 25;
  static constexpr int LDS_SLOT = (DL_ROW + 1) * ROW;
  static constexpr int DL_INDEX = DL_ROW * ROW;
  static __device__ __forceinline__ int slot_index(int p) {
    if (p < oW2) return (p / D1) * ROW + p % D1;
    if (p < oB2) return W2_ROW * ROW + (p - oW2);
    return D0 * ROW + D1;
  }
  template <int LIK>
  __device__ __forceinline__ float finish(int p, float v, const float* s_w) const {
    const float gr = LIK == 1 ? ratio : 1.0f;
    if (p < oW2) return v * (4.0f * gr * s_w[oW2 + p % D1]);
    return v * gr;  // layer-2 weights and b2
  }

  template <int LIK>
  __device__ __forceinline__ void write_partials(float* slot, const float*, bool last) {
    const int lane = opaque_tid() & 63, n = lane & 15, q = lane >> 4, r = n & 3, cb = n >> 2;
    // The lane swaps below read the accumulators from inside assembly statements, where the compiler does not
    // count the wait states a vector instruction needs after a matrix instruction wrote its operand (up to 11
    // for the wide ones).  Once per step: sixteen wait states here cover whatever the tile loop ended on.
    asm volatile("s_nop 15" ::: "memory");
    // ---- hidden 0 .. 31, features 0 .. 15: lane (n, q), component i: c = 16 t + 4 q + i, f = n ----
#pragma unroll
    for (int t = 0; t < NT; ++t) *reinterpret_cast<f4*>(slot + n * ROW + 16 * t + 4 * q) = dacc_e[t];
    // ---- hidden 0 .. 31, features 16 .. 23 (as MfmaLayer::write_partials): after the folds the lane holds
    //      c = 16 t + 4 cb + (q & 1) + 2 h and f = 16 + 2 r + (q >> 1) ----
    {
      const int c0 = 4 * cb + (q & 1);
      const int f = 16 + 2 * r + (q >> 1);
#pragma unroll
      for (int t = 0; t < NT; ++t) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const float v = fold4(dacc_f[t][0][2 * h], dacc_f[t][1][2 * h], dacc_f[t][0][2 * h + 1],
                                dacc_f[t][1][2 * h + 1]);
          slot[f * ROW + 16 * t + c0 + 2 * h] = v;
        }
      }
    }
    // ---- hidden 32 .. 39: d5[fs][i] is a partial over the row groups q and the row pairs h8.  fold4 over the
    //      four components leaves row q of lanes with the sum over q of component i(q) = 2 (q & 1) + (q >> 1);
    //      adding lane n ^ 8 sums the two row pairs ----
    {
      const int c = 32 + 4 * (cb & 1) + 2 * (q & 1) + (q >> 1);
#pragma unroll
      for (int fs = 0; fs < 6; ++fs) {
        float v = fold4(d5[fs][0], d5[fs][1], d5[fs][2], d5[fs][3]);
        v += dpp_move<0x128>(v);  // row_ror:8
        slot[(6 * r + fs) * ROW + c] = v;  // (lanes n and n ^ 8 store the same bits to the same place)
      }
    }
    // ---- dw2 = sum g h = 2 sum g (s - 1/2): hidden 0 .. 31 as 2 (dw2s - hs), hidden 32 .. 39 as 2 dw2s5;
    //      db2 = sum g = 2 hs.  Row q of lanes ends with: q = 0 hidden n, q = 2 hidden 16 + n, q = 1 and 3
    //      hidden 32 + c8 (lanes n and n ^ 8, rows 1 and 3 store the same bits to the same place) ----
    {
      float d5s = dw2s5;
      d5s += dpp_move<0x128>(d5s);
      const float v = fold4(2.0f * (dw2s[0] - hs), 2.0f * (dw2s[1] - hs), 2.0f * d5s, 2.0f * d5s);
      const int col = q == 0 ? n : (q == 2 ? 16 + n : 32 + (n & 7));
      slot[W2_ROW * ROW + col] = v;
      const float g2 = fold4(hs, hs, hs, hs);  // every lane: the sum over the wave's rows of g / 2
      if (lane == 0) slot[D0 * ROW + D1] = 2.0f * g2;
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
