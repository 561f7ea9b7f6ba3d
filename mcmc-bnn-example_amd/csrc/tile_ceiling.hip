// Ceiling of the tile loop of the 22 -> 40 -> 1 MFMA trajectory kernel on gfx950: the tile's own
// instruction mix -- GEMM1 (18 MFMAs 16x16x4), the pointwise stage, GEMM2 (12 MFMAs 16x16x4 and
// 24 MFMAs 4x4x1), taken from the very header the kernel is built from -- run on registers, with no memory traffic, no barrier and no
// reduction, two waves per SIMD as in the kernel.  FP32 MFMA and vector instructions share one pipe
// on this chip, so the time per tile is what that instruction mix costs on it; the production loop can
// come close to this number but not beat it.  Also times the two halves of the mix alone, and two
// alternative mixes in which the eight hidden units beyond the second 16-wide hidden tile (32 .. 39) leave
// the half-empty third tile for 4x4x1 blocks (see hybrid_kernel below).  Then the same for the tile of the
// 64 -> 128 -> 1 kernel (256 v_mfma_f32_16x16x4_f32 per 16-row tile, the W1 operand read from LDS, one wave
// per SIMD as in that kernel): whole tile, matrix instructions alone, pointwise stage alone.
//
//   tile_ceiling [tiles per wave]      (default 30000; the 64 -> 128 -> 1 tile runs a fifth of them)
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

#include "bnn_mfma_hybrid_layer.h"
#include "bnn_mfma_layer.h"
#include "bnn_mfma_wide_layer.h"

using namespace bnn;
using Layer = MfmaLayer<22, 40, 2>;

// MODE 0: the whole tile; 1: the MFMAs alone; 2: the pointwise stage alone
template <int MODE>
__global__ __launch_bounds__(512) void tile_kernel(float* out, unsigned long long* cycles, int tiles,
                                                   ModelConsts mc, const float* w) {
  __shared__ float s_w[Layer::P_AL];
  for (int p = threadIdx.x; p < Layer::P; p += blockDim.x) s_w[p] = w[p];
  __syncthreads();
  const int lane = threadIdx.x & 63, n = lane & 15, q = lane >> 4;
  Layer layer;
  layer.load_weights<1>(s_w, mc);
  layer.zero_acc();
  StepCtx cx;
  cx.n = 1 << 30;
  cx.ell_prev = nullptr;
  cx.ell_new = nullptr;
  Layer::TileIn ti;
  for (int i = 0; i < Layer::KP; ++i) ti.xa[i] = f2{0.01f * (lane + i), -0.02f * (lane - i)};
  for (int j = 0; j < 4; ++j) {
    ti.xe[j] = 0.02f * (n - j);
    ti.xf[j] = f2{0.03f * (n + j), 0.01f * (q - j)};
  }
  ti.y1 = 0.1f * q;
  f4 acc[Layer::NT];
  for (int t = 0; t < Layer::NT; ++t) acc[t] = f4{0.1f * n, -0.2f, 0.3f, 0.05f * q};
  const unsigned long long c0 = __builtin_readcyclecounter();
  const unsigned long long r0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < tiles; ++it) {
    // a new tile: the compiler must take the operands as unknown
    asm volatile("" : "+v"(ti.xa[0]), "+v"(ti.xa[1]), "+v"(ti.xa[2]), "+v"(ti.xe[0]), "+v"(ti.xe[1]),
                      "+v"(ti.xe[2]), "+v"(ti.xe[3]), "+v"(ti.xf[0]), "+v"(ti.xf[1]), "+v"(ti.xf[2]),
                      "+v"(ti.xf[3]), "+v"(ti.y1));
    float ge[4];
    f2 gf[4];
    if (MODE != 2) {
      layer.gemm1(ti.xa, acc);
    } else {
      asm volatile("" : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]));
    }
    if (MODE != 1) {
      layer.pointwise<1, false, true>(acc, ti, ge, gf, cx, mc, 0, n, q);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        ge[j] = ti.xe[j];
        gf[j] = ti.xf[j];
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (MODE != 2) {
      layer.gemm2(acc, ge, gf);
    } else {
      asm volatile("" ::"v"(ge[0]), "v"(ge[1]), "v"(ge[2]), "v"(ge[3]), "v"(gf[0]), "v"(gf[1]), "v"(gf[2]),
                   "v"(gf[3]), "v"(acc[0]), "v"(acc[1]), "v"(acc[2]));
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  const unsigned long long c1 = __builtin_readcyclecounter();
  float sum = 0.0f;
  for (int t = 0; t < Layer::NT; ++t) {
    sum += layer.dw2s[t];
    for (int j = 0; j < 4; ++j) sum += layer.dacc_e[t][j] + layer.dacc_f[t][0][j] + layer.dacc_f[t][1][j];
  }
  out[blockIdx.x * blockDim.x + threadIdx.x] = sum;
  if (threadIdx.x == 0) {
    cycles[2 * blockIdx.x] = c1 - c0;                                   // shader-clock ticks
    cycles[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - r0;  // 100 MHz ticks
  }
}

// ------------------------------------------------------------------------------------------------
// Alternative mixes: hidden units 32 .. 39 on v_mfma_f32_4x4x1_16b_f32 (sixteen independent 4x4 blocks).
//
// GEMM1, third hidden tile.  Block b = 4 q + cb (lanes 4 b .. 4 b + 3), twelve instructions s = 0 .. 11:
//     A_b[i] = x_aug[row 4 q + i][k = 12 (cb >> 1) + s]            (lane n = 4 cb + i supplies it)
//     B_b[r] = W1_aug[k][hidden 32 + 4 (cb & 1) + r]                (lane n = 4 cb + r)
//     D: lane (n, q), register i: row 4 q + i, hidden 32 + (n & 7), partial over the k-half n >> 3
//   i.e. the C layout of the 16-wide tiles, except that lanes n >= 8 hold the second half of the
//   contraction instead of eight padded hidden units: 12 x 8.4 cycles instead of 6 x 32.
// HYBRID == 1 ("GEMM1 only"): both halves are added into every lane (4 DPP additions, lanes n and n ^ 8 then
//   hold the same total) and the pointwise stage and GEMM2 go on as in production, whose third tile treats
//   lanes n >= 8 as padding; the sum of g, which production takes from a padded unit, costs one addition.
// HYBRID == 2 ("both GEMMs"): lanes n < 8 keep the totals of rows 4 q, 4 q + 1, lanes n >= 8 those of rows
//   4 q + 2, 4 q + 3 (4 bank-masked DPP additions): the pointwise stage runs on 10 values per lane instead of
//   12; g is folded into the A operand of GEMM2 (u g: 12 multiplications, none on the rows of x); GEMM2 of
//   the third tile is 12 blocks instructions  A_b[i] = u g of hidden 32 + 4 (cb & 1) + i, row R = 4 q +
//   2 (cb >> 1) + rho,  B_b[r] = x_aug[R][feature 6 r + fs]  (fs = 0 .. 5), instead of 4 wide and 8 block
//   instructions.
// Both need operands in layouts the production tile does not load: 12 floats per lane and tile for GEMM1
// (x_aug[row 4 q + (n & 3)][12 (n >> 3) ..+12]) and, for HYBRID == 2, 12 more for GEMM2.  Here they sit in
// registers: what is timed is the arithmetic alone.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ f4 mfma4(float a, float b, f4 c) { return __builtin_amdgcn_mfma_f32_4x4x1f32(a, b, c, 0, 0, 0); }
__device__ __forceinline__ f4 mfma16(float a, float b, f4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }

template <int HYBRID>
__global__ __launch_bounds__(512) void hybrid_kernel(float* out, unsigned long long* cycles, int tiles,
                                                     ModelConsts mc, const float* w) {
  __shared__ float s_w[Layer::P_AL];
  for (int p = threadIdx.x; p < Layer::P; p += blockDim.x) s_w[p] = w[p];
  __syncthreads();
  const int lane = threadIdx.x & 63, n = lane & 15, q = lane >> 4;
  Layer layer;
  layer.load_weights<1>(s_w, mc);
  layer.zero_acc();
  StepCtx cx;
  cx.n = 1 << 30;
  cx.ell_prev = nullptr;
  cx.ell_new = nullptr;
  Layer::TileIn ti;
  for (int i = 0; i < Layer::KP; ++i) ti.xa[i] = f2{0.01f * (lane + i), -0.02f * (lane - i)};
  for (int j = 0; j < 4; ++j) {
    ti.xe[j] = 0.02f * (n - j);
    ti.xf[j] = f2{0.03f * (n + j), 0.01f * (q - j)};
  }
  ti.y1 = 0.1f * q;
  float x5a[12], w5[12], x5b[2][6];
  for (int s = 0; s < 12; ++s) {
    x5a[s] = 0.01f * (lane - 3 * s);
    w5[s] = 0.02f * (n + s) - 0.3f;
    x5b[s / 6][s % 6] = 0.015f * (lane + s);
  }
  const float w2g5 = layer.w2g[2];
  f4 d5[6];
  for (int fs = 0; fs < 6; ++fs) d5[fs] = f4{0.f, 0.f, 0.f, 0.f};
  float dw2s5 = 0.0f, gsum = 0.0f;
  const unsigned long long c0 = __builtin_readcyclecounter();
  const unsigned long long r0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < tiles; ++it) {
    asm volatile("" : "+v"(ti.xa[0]), "+v"(ti.xa[1]), "+v"(ti.xa[2]), "+v"(ti.xe[0]), "+v"(ti.xe[1]),
                      "+v"(ti.xe[2]), "+v"(ti.xe[3]), "+v"(ti.xf[0]), "+v"(ti.xf[1]), "+v"(ti.xf[2]),
                      "+v"(ti.xf[3]), "+v"(ti.y1));
    asm volatile("" : "+v"(x5a[0]), "+v"(x5a[1]), "+v"(x5a[2]), "+v"(x5a[3]), "+v"(x5a[4]), "+v"(x5a[5]),
                      "+v"(x5a[6]), "+v"(x5a[7]), "+v"(x5a[8]), "+v"(x5a[9]), "+v"(x5a[10]), "+v"(x5a[11]));
    if (HYBRID == 2)
      asm volatile("" : "+v"(x5b[0][0]), "+v"(x5b[0][1]), "+v"(x5b[0][2]), "+v"(x5b[0][3]), "+v"(x5b[0][4]),
                        "+v"(x5b[0][5]), "+v"(x5b[1][0]), "+v"(x5b[1][1]), "+v"(x5b[1][2]), "+v"(x5b[1][3]),
                        "+v"(x5b[1][4]), "+v"(x5b[1][5]));
    // ---- GEMM1: hidden 0 .. 31 on two 16-wide tiles, hidden 32 .. 39 on 4x4 blocks ----
    f4 acc[3] = {f4{0.f, 0.f, 0.f, 0.f}, f4{0.f, 0.f, 0.f, 0.f}, f4{0.f, 0.f, 0.f, 0.f}};
    // (one block instruction after every wide one: the twelve block instructions accumulate into one register
    // quadruple and each needs its predecessor's result)
#pragma unroll
    for (int i = 0; i < Layer::KP; ++i) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        acc[0] = mfma16(ti.xa[i][h], layer.w1b[2 * i + h][0], acc[0]);
        acc[2] = mfma4(x5a[4 * i + 2 * h], w5[4 * i + 2 * h], acc[2]);
        acc[1] = mfma16(ti.xa[i][h], layer.w1b[2 * i + h][1], acc[1]);
        acc[2] = mfma4(x5a[4 * i + 2 * h + 1], w5[4 * i + 2 * h + 1], acc[2]);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (HYBRID == 1) {
      // both k-halves into every lane, then the production stages
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[2][j] += dpp_move<0x128>(acc[2][j]);  // row_ror:8
      float ge[4];
      f2 gf[4];
      layer.pointwise<1, false, true>(acc, ti, ge, gf, cx, mc, 0, n, q);
      gsum += ge[0];  // stands for the one addition that collects the sum of g
      __builtin_amdgcn_sched_barrier(0);
      layer.gemm2(acc, ge, gf);
      __builtin_amdgcn_sched_barrier(0);
      continue;
    }
    // ---- HYBRID == 2 ----
    // lanes n < 8: rows 4 q, 4 q + 1 (registers 0, 1); lanes n >= 8: rows 4 q + 2, 4 q + 3 (registers 2, 3)
    float sa = acc[2][2], sb = acc[2][3];
    asm volatile("s_nop 7\n\t"
                 "v_add_f32_dpp %[a], %[a], %[a] row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                 "v_add_f32_dpp %[b], %[b], %[b] row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                 "v_add_f32_dpp %[a], %[p0], %[p0] row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
                 "v_add_f32_dpp %[b], %[p1], %[p1] row_ror:8 row_mask:0xf bank_mask:0x3"
                 : [a] "+v"(sa), [b] "+v"(sb)
                 : [p0] "v"(acc[2][0]), [p1] "v"(acc[2][1]));
    float yh[4] = {layer.y_0, layer.y_0, layer.y_0, layer.y_0};
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float e = __builtin_amdgcn_exp2f(acc[t][j]);
        const float sg = __builtin_amdgcn_rcpf(1.0f + e);
        acc[t][j] = sg;
        yh[j] = __builtin_fmaf(layer.w2g[t], sg, yh[j]);
      }
    }
    sa = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(sa));
    sb = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(sb));
    // the third tile's terms of the row sums: each lane holds two of its four rows
    asm volatile("s_nop 1\n\t"
                 "v_fmac_f32_dpp %[y0], %[a], %[w] quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0x3\n\t"
                 "v_fmac_f32_dpp %[y2], %[a], %[w] quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0xc\n\t"
                 "v_fmac_f32_dpp %[y1], %[b], %[w] quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0x3\n\t"
                 "v_fmac_f32_dpp %[y3], %[b], %[w] quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0xc"
                 : [y0] "+v"(yh[0]), [y1] "+v"(yh[1]), [y2] "+v"(yh[2]), [y3] "+v"(yh[3])
                 : [a] "v"(sa), [b] "v"(sb), [w] "v"(w2g5));
    const float gz = row16_reduce4(yh[0], yh[1], yh[2], yh[3]) + __builtin_fmaf(ti.y1, layer.k2v, layer.rho);
    gsum += gz;
    // dw2s += g s  and  u g = (s - s^2) g, g of row 4 q + j read from bank j of gz
    float ug[2][4], uga, ugb;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int j = 0; j < 4; ++j) ug[t][j] = __builtin_fmaf(-acc[t][j], acc[t][j], acc[t][j]);
    }
    uga = __builtin_fmaf(-sa, sa, sa);
    ugb = __builtin_fmaf(-sb, sb, sb);
#define BNN_BC(j) " row_newbcast:" #j " row_mask:0xf bank_mask:0xf\n\t"
    asm volatile("s_nop 1\n\t"
                 "v_fmac_f32_dpp %[d0], %[g], %[s00]" BNN_BC(0)
                 "v_fmac_f32_dpp %[d1], %[g], %[s10]" BNN_BC(0)
                 "v_fmac_f32_dpp %[d0], %[g], %[s01]" BNN_BC(4)
                 "v_fmac_f32_dpp %[d1], %[g], %[s11]" BNN_BC(4)
                 "v_fmac_f32_dpp %[d0], %[g], %[s02]" BNN_BC(8)
                 "v_fmac_f32_dpp %[d1], %[g], %[s12]" BNN_BC(8)
                 "v_fmac_f32_dpp %[d0], %[g], %[s03]" BNN_BC(12)
                 "v_fmac_f32_dpp %[d1], %[g], %[s13]" BNN_BC(12)
                 "v_fmac_f32_dpp %[d5], %[g], %[sa] row_newbcast:0 row_mask:0xf bank_mask:0x3\n\t"
                 "v_fmac_f32_dpp %[d5], %[g], %[sa] row_newbcast:8 row_mask:0xf bank_mask:0xc\n\t"
                 "v_fmac_f32_dpp %[d5], %[g], %[sb] row_newbcast:4 row_mask:0xf bank_mask:0x3\n\t"
                 "v_fmac_f32_dpp %[d5], %[g], %[sb] row_newbcast:12 row_mask:0xf bank_mask:0xc"
                 : [d0] "+v"(layer.dw2s[0]), [d1] "+v"(layer.dw2s[1]), [d5] "+v"(dw2s5)
                 : [g] "v"(gz), [s00] "v"(acc[0][0]), [s01] "v"(acc[0][1]), [s02] "v"(acc[0][2]), [s03] "v"(acc[0][3]),
                   [s10] "v"(acc[1][0]), [s11] "v"(acc[1][1]), [s12] "v"(acc[1][2]), [s13] "v"(acc[1][3]),
                   [sa] "v"(sa), [sb] "v"(sb));
    asm volatile("s_nop 1\n\t"
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
    // ---- GEMM2: hidden 0 .. 31 as in production (g now rides on A), hidden 32 .. 39 on 4x4 blocks ----
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      layer.dacc_e[0] = mfma16(ug[0][j], ti.xe[j], layer.dacc_e[0]);
      layer.dacc_e[1] = mfma16(ug[1][j], ti.xe[j], layer.dacc_e[1]);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        layer.dacc_f[t][0] = mfma4(ug[t][j], ti.xf[j][0], layer.dacc_f[t][0]);
        layer.dacc_f[t][1] = mfma4(ug[t][j], ti.xf[j][1], layer.dacc_f[t][1]);
      }
    }
#pragma unroll
    for (int fs = 0; fs < 6; ++fs) {
      d5[fs] = mfma4(uga, x5b[0][fs], d5[fs]);
      d5[fs] = mfma4(ugb, x5b[1][fs], d5[fs]);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  const unsigned long long c1 = __builtin_readcyclecounter();
  float sum = dw2s5 + gsum;
  for (int fs = 0; fs < 6; ++fs)
    for (int j = 0; j < 4; ++j) sum += d5[fs][j];
  for (int t = 0; t < Layer::NT; ++t) {
    sum += layer.dw2s[t];
    for (int j = 0; j < 4; ++j) sum += layer.dacc_e[t][j] + layer.dacc_f[t][0][j] + layer.dacc_f[t][1][j];
  }
  out[blockIdx.x * blockDim.x + threadIdx.x] = sum;
  if (threadIdx.x == 0) {
    cycles[2 * blockIdx.x] = c1 - c0;
    cycles[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - r0;
  }
}

// ------------------------------------------------------------------------------------------------
// The tile the kernel runs by default: MfmaHybridLayer::compute_tile (hidden 32 .. 39 on 4x4 blocks in both
// contractions, the block operands read from the wave's LDS copy of the tile), on a tile held in registers.
// ------------------------------------------------------------------------------------------------
using Hybrid = MfmaHybridLayer<22, 40>;
__global__ __launch_bounds__(512) void hybrid_layer_kernel(float* out, unsigned long long* cycles, int tiles,
                                                           ModelConsts mc, const float* w) {
  __shared__ float s_w[Hybrid::P_AL];
  __shared__ __align__(16) float s_tile[8][Hybrid::TILE_LDS];
  for (int p = threadIdx.x; p < Hybrid::P; p += blockDim.x) s_w[p] = w[p];
  __syncthreads();
  const int lane = threadIdx.x & 63, n = lane & 15, q = lane >> 4;
  Hybrid layer;
  layer.load_weights<1>(s_w, mc);
  layer.zero_acc();
  StepCtx cx;
  cx.n = 1 << 30;
  cx.ell_prev = nullptr;
  cx.ell_new = nullptr;
  Hybrid::TileIn ti;
  for (int i = 0; i < Hybrid::KP; ++i) ti.xa[i] = f2{0.01f * (lane + i), -0.02f * (lane - i)};
  ti.y1 = 0.1f * q;
  float* tile = s_tile[threadIdx.x >> 6];
  const unsigned long long c0 = __builtin_readcyclecounter();
  const unsigned long long r0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < tiles; ++it) {
    asm volatile("" : "+v"(ti.xa[0]), "+v"(ti.xa[1]), "+v"(ti.xa[2]), "+v"(ti.y1));
    layer.compute_tile<1, false, true>(ti, tile, cx, mc, 0, n, q);
  }
  const unsigned long long c1 = __builtin_readcyclecounter();
  float sum = layer.dw2s5 + layer.hs;
  for (int fs = 0; fs < 6; ++fs)
    for (int j = 0; j < 4; ++j) sum += layer.d5[fs][j];
  for (int t = 0; t < Hybrid::NT; ++t) {
    sum += layer.dw2s[t];
    for (int j = 0; j < 4; ++j) sum += layer.dacc_e[t][j] + layer.dacc_f[t][0][j] + layer.dacc_f[t][1][j];
  }
  out[blockIdx.x * blockDim.x + threadIdx.x] = sum;
  if (threadIdx.x == 0) {
    cycles[2 * blockIdx.x] = c1 - c0;
    cycles[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - r0;
  }
}

// ------------------------------------------------------------------------------------------------
// The tile of the 64 -> 128 -> 1 kernel: MfmaWideLayer::compute_tile on a tile held in registers, the
// weights in LDS as in the kernel, 256 threads per workgroup = one wave per SIMD.
// ------------------------------------------------------------------------------------------------
// Two tiles per trip with nothing between them, as in the kernel's loop (the compiler may overlap the end
// of one tile with the start of the next).
using WideLayer = MfmaWideLayer<64, 128>;
template <int PARTS>
__global__ __launch_bounds__(256) void wide_kernel(float* out, unsigned long long* cycles, int tiles,
                                                   ModelConsts mc, const float* w) {
  __shared__ __align__(16) float s_w[WideLayer::P_AL];
  for (int p = threadIdx.x; p < WideLayer::P; p += blockDim.x) s_w[p] = w[p % Layer::P];
  __syncthreads();
  const int lane = threadIdx.x & 63, n = lane & 15, q = lane >> 4;
  WideLayer layer;
  layer.prepare_step(s_w, mc);
  layer.zero_acc();
  StepCtx cx;
  cx.n = 1 << 30;
  cx.ell_prev = nullptr;
  cx.ell_new = nullptr;
  WideLayer::Tile ti;
  for (int i = 0; i < WideLayer::KQ; ++i) ti.xa[i] = f4{0.01f * (lane + i), -0.02f * (lane - i), 0.03f * i, 0.01f * q};
  for (int j = 0; j < 4; ++j)
    for (int v = 0; v < WideLayer::FV; ++v) ti.xb[j][v] = f2{0.03f * (n + j), 0.01f * (q - j + v)};
  ti.y1 = 0.1f * q;
  const unsigned long long c0 = __builtin_readcyclecounter();
  const unsigned long long r0 = __builtin_amdgcn_s_memrealtime();
  WideLayer::Tile tj = ti;
  auto opaque = [](WideLayer::Tile& t) {
    asm volatile("" : "+v"(t.xa[0]), "+v"(t.xa[1]), "+v"(t.xa[2]), "+v"(t.xa[3]), "+v"(t.xb[0][0]),
                      "+v"(t.xb[0][1]), "+v"(t.xb[1][0]), "+v"(t.xb[1][1]), "+v"(t.xb[2][0]),
                      "+v"(t.xb[2][1]), "+v"(t.xb[3][0]), "+v"(t.xb[3][1]), "+v"(t.y1));
  };
  for (int it = 0; it < tiles; it += 2) {
    opaque(ti);
    opaque(tj);
    layer.compute_tile<1, false, true, PARTS>(ti, s_w, cx, mc, 0, n, q);
    layer.compute_tile<1, false, true, PARTS>(tj, s_w, cx, mc, 16, n, q);
  }
  const unsigned long long c1 = __builtin_readcyclecounter();
  float sum = layer.db2acc;
  for (int t = 0; t < WideLayer::NT; ++t) {
    sum += layer.dw2acc[t] + layer.db1acc[t];
    for (int ft = 0; ft < WideLayer::FT; ++ft)
      for (int j = 0; j < 4; ++j) sum += layer.dacc[t][ft][j];
  }
  out[blockIdx.x * blockDim.x + threadIdx.x] = sum;
  if (threadIdx.x == 0) {
    cycles[2 * blockIdx.x] = c1 - c0;
    cycles[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - r0;
  }
}

#define HIP_CHECK(x)                                                                    \
  do {                                                                                  \
    hipError_t e_ = (x);                                                                \
    if (e_ != hipSuccess) {                                                             \
      std::fprintf(stderr, "%s failed: %s (%s:%d)\n", #x, hipGetErrorString(e_), __FILE__, __LINE__); \
      return 1;                                                                         \
    }                                                                                   \
  } while (0)

typedef void (*TileKernel)(float*, unsigned long long*, int, ModelConsts, const float*);
int run(TileKernel kernel, const char* what, int tiles, float* d_out, unsigned long long* d_cyc,
        const ModelConsts& mc, const float* d_w, int threads = 512) {
  const int wgs = 256;
  hipEvent_t e0, e1;
  HIP_CHECK(hipEventCreate(&e0));
  HIP_CHECK(hipEventCreate(&e1));
  // warm-up long enough for the clocks to settle
  hipLaunchKernelGGL(kernel, dim3(wgs), dim3(threads), 0, 0, d_out, d_cyc, 10 * tiles, mc, d_w);
  HIP_CHECK(hipDeviceSynchronize());
  HIP_CHECK(hipEventRecord(e0));
  hipLaunchKernelGGL(kernel, dim3(wgs), dim3(threads), 0, 0, d_out, d_cyc, tiles, mc, d_w);
  HIP_CHECK(hipEventRecord(e1));
  HIP_CHECK(hipEventSynchronize(e1));
  float ms = 0;
  HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
  std::vector<unsigned long long> cyc(2 * wgs);
  HIP_CHECK(hipMemcpy(cyc.data(), d_cyc, cyc.size() * sizeof(cyc[0]), hipMemcpyDeviceToHost));
  double mean = 0, real = 0;
  for (int i = 0; i < wgs; ++i) {
    mean += (double)cyc[2 * i] / wgs;
    real += (double)cyc[2 * i + 1] / wgs;
  }
  // A SIMD holds threads / 256 waves (two in the 22 -> 40 -> 1 kernel, where it issues the older one first,
  // so a wave's own start-to-end ticks say little); the launch as a whole takes that many times `tiles` tiles
  // per SIMD, and the shader clock is the ratio of the two counters that one wave read.
  const double mhz = mean / (real * 1e-2);
  std::printf("%-36s %9.3f ms (events), shader clock %.0f MHz, %8.1f cycles per tile and SIMD\n", what, ms, mhz,
              ms * 1e-3 * mhz * 1e6 / ((threads / 256) * (double)tiles));
  return 0;
}

int main(int argc, char** argv) {
  const int tiles = argc > 1 ? std::atoi(argv[1]) : 30000;
  ModelConsts mc{};
  mc.scale = 0.01f;
  mc.scale_recp = 100.0f;
  mc.df = 2.2f;
  mc.df_recp = 1.0f / 2.2f;
  mc.prior_recp = 10.0f;
  std::vector<float> w(Layer::P);
  for (int p = 0; p < Layer::P; ++p) w[p] = 0.05f * (float)((p * 37) % 41 - 20) / 20.0f;
  float *d_out = nullptr, *d_w = nullptr;
  unsigned long long* d_cyc = nullptr;
  HIP_CHECK(hipMalloc((void**)&d_out, 256 * 512 * sizeof(float)));
  HIP_CHECK(hipMalloc((void**)&d_w, w.size() * sizeof(float)));
  HIP_CHECK(hipMalloc((void**)&d_cyc, 2 * 256 * sizeof(unsigned long long)));
  HIP_CHECK(hipMemcpy(d_w, w.data(), w.size() * sizeof(float), hipMemcpyHostToDevice));
  std::printf("tile of 16 rows, 22 -> 40 -> 1, two waves per SIMD, %d tiles per wave, 256 workgroups of 512 threads\n",
              tiles);
  if (run(tile_kernel<0>, "whole tile (MFMAs + pointwise)", tiles, d_out, d_cyc, mc, d_w)) return 1;
  if (run(tile_kernel<1>, "the MFMAs alone", tiles, d_out, d_cyc, mc, d_w)) return 1;
  if (run(tile_kernel<2>, "the pointwise stage alone", tiles, d_out, d_cyc, mc, d_w)) return 1;
  if (run(hybrid_kernel<1>, "hidden 32..39 on 4x4 blocks: GEMM1", tiles, d_out, d_cyc, mc, d_w)) return 1;
  if (run(hybrid_kernel<2>, "hidden 32..39 on 4x4 blocks: both", tiles, d_out, d_cyc, mc, d_w)) return 1;
  if (run(hybrid_layer_kernel, "the same as the kernel runs it (LDS)", tiles, d_out, d_cyc, mc, d_w)) return 1;
  const int wt = tiles / 5 > 0 ? tiles / 5 : 1;
  std::printf("tile of 16 rows, 64 -> 128 -> 1, one wave per SIMD, %d tiles per wave, 256 workgroups of 256 threads\n", wt);
  if (run(wide_kernel<3>, "whole tile (MFMAs + pointwise)", wt, d_out, d_cyc, mc, d_w, 256)) return 1;
  if (run(wide_kernel<1>, "the MFMAs and their LDS operand reads", wt, d_out, d_cyc, mc, d_w, 256)) return 1;
  if (run(wide_kernel<2>, "the pointwise stage alone", wt, d_out, d_cyc, mc, d_w, 256)) return 1;
  return 0;
}
