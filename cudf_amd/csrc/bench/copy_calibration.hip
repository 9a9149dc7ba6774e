// Plain device-to-device copy of a known size, used to calibrate the HBM traffic counters
// (FETCH_SIZE / WRITE_SIZE of rocprofv3 --pmc) that are quoted for the library's kernels: the factor
// between what a counter reads for this kernel and the bytes it is known to move scales the other readings.
// A second kernel reads 32-byte records (a bucket of the tokenizer's table) at scattered places of a table far larger
// than the caches, so that every read goes to memory: what FETCH_SIZE counts for it, times the copy kernel's factor,
// is the price of one such read in that counter's bytes (32 would be the bytes asked for, 64 or 128 the size of what
// memory hands over per request).
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

__global__ void __launch_bounds__(256) scattered_read_calibration_kernel(const uint4* __restrict__ table, uint32_t record_mask, uint32_t reads_per_thread,
                                                                        uint32_t* __restrict__ out)
{
  uint32_t const t = blockIdx.x * blockDim.x + threadIdx.x;
  uint32_t x       = t * 0x9E3779B1u + 0x7F4A7C15u;
  uint32_t acc     = 0;
  for (uint32_t i = 0; i < reads_per_thread; ++i) {
    x ^= x << 13;
    x ^= x >> 17;
    x ^= x << 5;
    uint32_t const r = (x * 0x85EBCA77u >> 4) & record_mask;  // a record of two uint4
    uint4 const a = table[2 * static_cast<size_t>(r)], b = table[2 * static_cast<size_t>(r) + 1];
    acc += a.x ^ a.w ^ b.y ^ b.z;
  }
  out[t] = acc;
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

  // scattered 32-byte reads: 2^25 of them per launch (1 GiB asked for) from tables of 4 GiB and of 16 MiB
  for (int which = 0; which < 2; ++which) {
    size_t const table_bytes = which == 0 ? (size_t{4} << 30) : (size_t{16} << 20);
    uint4* table             = nullptr;
    uint32_t* out            = nullptr;
    uint32_t const threads = 1u << 20, per_thread = 32;
    CHECK(hipMalloc(&table, table_bytes));
    CHECK(hipMalloc(&out, threads * sizeof(uint32_t)));
    CHECK(hipMemset(table, 0x3c, table_bytes));
    for (int i = 0; i < launches + 1; ++i) {
      if (i == 1) CHECK(hipEventRecord(t0, nullptr));
      hipLaunchKernelGGL(scattered_read_calibration_kernel, dim3(threads / 256), dim3(256), 0, nullptr, table, static_cast<uint32_t>(table_bytes / 32 - 1), per_thread, out);
    }
    CHECK(hipEventRecord(t1, nullptr));
    CHECK(hipDeviceSynchronize());
    CHECK(hipEventElapsedTime(&ms, t0, t1));
    printf("scattered_read_calibration_kernel: %zu reads of 32 bytes per launch (%zu bytes asked for) from a table of %zu MiB, %.3f ms per launch\n",
           static_cast<size_t>(threads) * per_thread, static_cast<size_t>(threads) * per_thread * 32, table_bytes >> 20, ms / launches);
    CHECK(hipFree(table));
    CHECK(hipFree(out));
  }
  return 0;
}
