// The MFMA layer of the 64 -> 128 -> 1 trajectory kernel: both contractions of a 16-row tile on
// v_mfma_f32_16x16x4_f32 with no padding, the pointwise stage between them, the tile loop and the wave's
// partial sums.  In a header of its own so that the tile-ceiling probe (tile_ceiling.hip) times exactly the
// code the kernel runs.
#pragma once

#include <hip/hip_runtime.h>

#include "bnn_device.h"
#include "bnn_kernel_common.h"

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

  // GEMM1 + activation + loss gradient + GEMM2 of one tile.  PARTS is for the tile-ceiling probe, which
  // times the halves of the instruction mix alone: 1 = the matrix instructions and their operand fetch
  // from LDS, 2 = the pointwise stage, 3 = the whole tile (what the kernel runs).
  template <int LIK, bool LAST, bool FULL, int PARTS = 3>
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
    if (PARTS & 1) {
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
    }
    if (PARTS == 2) {  // probe only: unknown pre-activations
#pragma unroll
      for (int t = 0; t < NT; ++t) asm volatile("" : "+v"(acc[t]));
    }
    f2 gx[4][FV];
    if (PARTS & 2) {
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
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int v = 0; v < FV; ++v) gx[j][v] = ti.xb[j][v] * g[j];
      }
    } else {  // probe only: the matrix instructions on the raw operands
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int v = 0; v < FV; ++v) gx[j][v] = ti.xb[j][v];
      }
    }
    if (PARTS & 1) {
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
    } else {  // probe only: keep the pointwise stage's results alive
#pragma unroll
      for (int t = 0; t < NT; ++t) asm volatile("" ::"v"(acc[t]));
#pragma unroll
      for (int j = 0; j < 4; ++j) asm volatile("" ::"v"(gx[j][0]), "v"(gx[j][1]));
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

}  // namespace bnn
