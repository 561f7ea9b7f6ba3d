// Plain device-to-device copy kernel of a known size, used to calibrate the FETCH_SIZE / WRITE_SIZE
// hardware counters: run it under `rocprofv3 --pmc FETCH_SIZE` (or WRITE_SIZE) and compare the counter
// with the bytes printed here.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

__global__ void copy_kernel(const float4* __restrict__ src, float4* __restrict__ dst, size_t n) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

int main(int argc, char** argv) {
  const size_t mib = argc > 1 ? (size_t)std::atol(argv[1]) : 1024;
  const size_t bytes = mib << 20, n = bytes / sizeof(float4);
  float4 *src = nullptr, *dst = nullptr;
  if (hipMalloc((void**)&src, bytes) != hipSuccess || hipMalloc((void**)&dst, bytes) != hipSuccess) {
    std::fprintf(stderr, "hipMalloc failed\n");
    return 1;
  }
  if (hipMemset(src, 1, bytes) != hipSuccess || hipMemset(dst, 0, bytes) != hipSuccess) return 1;
  if (hipDeviceSynchronize() != hipSuccess) return 1;
  hipLaunchKernelGGL(copy_kernel, dim3(256 * 8), dim3(256), 0, 0, src, dst, n);
  if (hipDeviceSynchronize() != hipSuccess) return 1;
  std::printf("copy_kernel moved %zu bytes in and %zu bytes out (%zu KiB each way)\n", bytes, bytes,
              bytes >> 10);
  (void)hipFree(src);
  (void)hipFree(dst);
  return 0;
}
