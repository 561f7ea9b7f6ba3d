// Ceiling of the tile loop of the 22 -> 40 -> 1 MFMA trajectory kernel on gfx950: the tile's own
// instruction mix -- GEMM1 (18 MFMAs 16x16x4), the pointwise stage, GEMM2 (12 MFMAs 16x16x4 and
// 24 MFMAs 4x4x1), taken from the very header the kernel is built from -- run on registers, with no memory traffic, no barrier and no
// reduction, two waves per SIMD as in the kernel.  FP32 MFMA and vector instructions share one pipe
// on this chip, so the time per tile is what that instruction mix costs on it; the production loop can
// come close to this number but not beat it.  Also times the two halves of the mix alone.
//
//   tile_ceiling [tiles per wave]      (default 30000)
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

#include "bnn_mfma_layer.h"

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

#define HIP_CHECK(x)                                                                    \
  do {                                                                                  \
    hipError_t e_ = (x);                                                                \
    if (e_ != hipSuccess) {                                                             \
      std::fprintf(stderr, "%s failed: %s (%s:%d)\n", #x, hipGetErrorString(e_), __FILE__, __LINE__); \
      return 1;                                                                         \
    }                                                                                   \
  } while (0)

template <int MODE>
int run(const char* what, int tiles, float* d_out, unsigned long long* d_cyc, const ModelConsts& mc,
        const float* d_w) {
  const int wgs = 256;
  hipEvent_t e0, e1;
  HIP_CHECK(hipEventCreate(&e0));
  HIP_CHECK(hipEventCreate(&e1));
  // warm-up long enough for the clocks to settle
  hipLaunchKernelGGL(tile_kernel<MODE>, dim3(wgs), dim3(512), 0, 0, d_out, d_cyc, 10 * tiles, mc, d_w);
  HIP_CHECK(hipDeviceSynchronize());
  HIP_CHECK(hipEventRecord(e0));
  hipLaunchKernelGGL(tile_kernel<MODE>, dim3(wgs), dim3(512), 0, 0, d_out, d_cyc, tiles, mc, d_w);
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
  // A SIMD holds two waves and issues the older one first, so a wave's own start-to-end ticks say little;
  // the launch as a whole takes 2 * tiles tiles per SIMD, and the shader clock is the ratio of the two
  // counters that one wave read.
  const double mhz = mean / (real * 1e-2);
  std::printf("%-34s %9.3f ms (events), shader clock %.0f MHz, %8.1f cycles per tile and SIMD\n", what, ms, mhz,
              ms * 1e-3 * mhz * 1e6 / (2.0 * tiles));
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
  if (run<0>("whole tile (MFMAs + pointwise)", tiles, d_out, d_cyc, mc, d_w)) return 1;
  if (run<1>("the MFMAs alone", tiles, d_out, d_cyc, mc, d_w)) return 1;
  if (run<2>("the pointwise stage alone", tiles, d_out, d_cyc, mc, d_w)) return 1;
  return 0;
}
