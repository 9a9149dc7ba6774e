// Plain device-to-device copy of a known size, used to calibrate the HBM traffic counters
// (FETCH_SIZE / WRITE_SIZE of rocprofv3 --pmc) that are quoted for the library's kernels: the factor
// between what a counter reads for this kernel and the bytes it is known to move scales the other readings.
// Build and run:
//   hipcc --offload-arch=gfx950 -O3 -o copy_calibration cudf_amd/csrc/bench/copy_calibration.hip && ./copy_calibration
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#define CHECK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s line %d\n", hipGetErrorString(e), __LINE__); return 1; } } while (0)

__global__ void __launch_bounds__(256) copy_calibration_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, size_t n)
{
  size_t const stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

int main()
{
  size_t const bytes = size_t{1} << 30;  // 1 GiB read + 1 GiB written per launch
  size_t const n     = bytes / sizeof(uint4);
  uint4 *src = nullptr, *dst = nullptr;
  CHECK(hipMalloc(&src, bytes));
  CHECK(hipMalloc(&dst, bytes));
  CHECK(hipMemset(src, 0x5a, bytes));
  CHECK(hipMemset(dst, 0, bytes));
  hipEvent_t t0, t1;
  CHECK(hipEventCreate(&t0));
  CHECK(hipEventCreate(&t1));
  int const launches = 5;
  for (int i = 0; i < launches + 1; ++i) {
    if (i == 1) CHECK(hipEventRecord(t0, nullptr));
    hipLaunchKernelGGL(copy_calibration_kernel, dim3(256 * 16), dim3(256), 0, nullptr, dst, src, n);
  }
  CHECK(hipEventRecord(t1, nullptr));
  CHECK(hipDeviceSynchronize());
  float ms = 0.f;
  CHECK(hipEventElapsedTime(&ms, t0, t1));
  printf("copy_calibration_kernel: %zu bytes read + %zu bytes written per launch, %.3f ms per launch, %.1f GB/s (read+write)\n", bytes, bytes,
         ms / launches, 2.0 * bytes / (ms / launches * 1e-3) / 1e9);
  CHECK(hipFree(src));
  CHECK(hipFree(dst));
  return 0;
}
