// Microbenchmark of the FP32 issue pipes of one SIMD on gfx950: how fast v_mfma_f32_16x16x4_f32,
// v_fma_f32 and v_exp_f32 issue alone, with two waves per SIMD, and when an MFMA wave and a VALU wave
// share a SIMD.  It answers whether FP32 MFMA work and ordinary vector work overlap (they do not:
// the mixed run takes the sum of the two separate times), which sets the achievable fraction of the
// FP32 roofline for a kernel that needs both.
#include <hip/hip_runtime.h>
#include <cstdio>
#define HIP_CHECK(x) do { if ((x) != hipSuccess) { std::fprintf(stderr, "HIP error at %s:%d\n", __FILE__, __LINE__); return 1; } } while (0)
typedef float f4 __attribute__((ext_vector_type(4)));
// 512 threads = 8 waves; wave w sits on SIMD w % 4.  role(wave) decides what the wave does.
// ROLE: 0 all MFMA; 1 all FMA; 2 waves 0-3 MFMA, waves 4-7 FMA (one of each per SIMD); 3 all EXP (trans); 4: waves 0-3 FMA, 4-7 EXP
// 5: waves 0-3 MFMA, 4-7 idle; 6: waves 0-3 FMA, 4-7 idle ; 7: waves 0-3 EXP, 4-7 idle; 8: waves 0-3 MFMA, 4-7 EXP
template <int ROLE>
__global__ __launch_bounds__(512) void k(float* out, int iters, float a, float b) {
  int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  int lo = wave < 4;
  int what; // 0 mfma 1 fma 2 exp 3 idle
  if (ROLE == 0) what = 0; else if (ROLE == 1) what = 1; else if (ROLE == 2) what = lo ? 0 : 1;
  else if (ROLE == 3) what = 2; else if (ROLE == 4) what = lo ? 1 : 2; else if (ROLE == 5) what = lo ? 0 : 3;
  else if (ROLE == 6) what = lo ? 1 : 3; else if (ROLE == 8) what = lo ? 0 : 2; else what = lo ? 2 : 3;
  f4 acc0 = {0,0,0,0}, acc1 = {0,0,0,0}, acc2={0,0,0,0}, acc3={0,0,0,0};
  float v[8];
  for (int i = 0; i < 8; ++i) v[i] = threadIdx.x * 0.001f + i;
  if (what == 0) {
    for (int it = 0; it < iters; ++it) {
      acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc0, 0,0,0);
      acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc1, 0,0,0);
      acc2 = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc2, 0,0,0);
      acc3 = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc3, 0,0,0);
    }
  } else if (what == 1) {
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = __builtin_fmaf(v[i], a, b);
    }
  } else if (what == 2) {
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = __builtin_amdgcn_exp2f(v[i]);
    }
  }
  float s = 0; for (int i = 0; i < 8; ++i) s += v[i];
  f4 t = acc0 + acc1 + acc2 + acc3;
  out[blockIdx.x * blockDim.x + threadIdx.x] = s + t[0] + t[1] + t[2] + t[3];
}
template <int ROLE>
float run(int iters, float* d) {
  hipEvent_t e0, e1;
  float ms = -1.0f;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return ms;
  hipLaunchKernelGGL((k<ROLE>), dim3(256), dim3(512), 0, 0, d, 10, 1.0f, 0.5f);
  if (hipDeviceSynchronize() != hipSuccess) return ms;
  (void)hipEventRecord(e0);
  hipLaunchKernelGGL((k<ROLE>), dim3(256), dim3(512), 0, 0, d, iters, 1.0f, 0.5f);
  (void)hipEventRecord(e1);
  (void)hipEventSynchronize(e1);
  (void)hipEventElapsedTime(&ms, e0, e1);
  return ms;
}
int main() {
  float* d = nullptr;
  HIP_CHECK(hipMalloc((void**)&d, 256 * 512 * 4));
  int iters = 100000;
  printf("per wave per iter: 4 MFMA 16x16x4 f32, or 32 v_fma_f32, or 32 v_exp_f32; iters=%d\n", iters);
  printf("1 wave/SIMD  MFMA        %.3f ms\n", run<5>(iters, d));
  printf("1 wave/SIMD  FMA         %.3f ms\n", run<6>(iters, d));
  printf("1 wave/SIMD  EXP         %.3f ms\n", run<7>(iters, d));
  printf("2 waves/SIMD MFMA+MFMA   %.3f ms\n", run<0>(iters, d));
  printf("2 waves/SIMD FMA+FMA     %.3f ms\n", run<1>(iters, d));
  printf("2 waves/SIMD EXP+EXP     %.3f ms\n", run<3>(iters, d));
  printf("2 waves/SIMD MFMA+FMA    %.3f ms\n", run<2>(iters, d));
  printf("2 waves/SIMD FMA+EXP     %.3f ms\n", run<4>(iters, d));
  printf("2 waves/SIMD MFMA+EXP    %.3f ms\n", run<8>(iters, d));
  return 0;
}
