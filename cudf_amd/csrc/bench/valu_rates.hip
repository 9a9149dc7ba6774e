// VALU instruction-rate probe for gfx950: each kernel runs a long unrolled chain of one instruction on 8
// independent registers per lane and reports wave-instructions per cycle per CU.  The minhash inner loop was
// chosen from these numbers.  Build and run:
//   hipcc --offload-arch=gfx950 -O3 -o valu_rates cudf_amd/csrc/bench/valu_rates.hip && ./valu_rates
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#define CHECK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s line %d\n", hipGetErrorString(e), __LINE__); return 1; } } while (0)
#define ITER 4096
#define DEF_KERNEL(NAME, ASM)                                                        \
  __global__ void NAME(uint32_t* out, uint32_t s) {                                  \
    uint32_t r0 = threadIdx.x, r1 = r0 + 1, r2 = r0 + 2, r3 = r0 + 3, r4 = r0 + 4, r5 = r0 + 5, r6 = r0 + 6, r7 = r0 + 7; \
    uint32_t x = s ^ threadIdx.x, y = s + 77;                                        \
    for (int i = 0; i < ITER; ++i) {                                                 \
      asm volatile(ASM(0) ASM(1) ASM(2) ASM(3) ASM(4) ASM(5) ASM(6) ASM(7)          \
                   : "+v"(r0), "+v"(r1), "+v"(r2), "+v"(r3), "+v"(r4), "+v"(r5), "+v"(r6), "+v"(r7) \
                   : "v"(x), "v"(y));                                                \
    }                                                                                \
    out[blockIdx.x * blockDim.x + threadIdx.x] = r0 ^ r1 ^ r2 ^ r3 ^ r4 ^ r5 ^ r6 ^ r7; \
  }
#define A_MULLO(i) "v_mul_lo_u32 %" #i ", %" #i ", %8\n"
#define A_MAD24(i) "v_mad_u32_u24 %" #i ", %" #i ", %8, %9\n"
#define A_MUL24(i) "v_mul_u32_u24 %" #i ", %" #i ", %8\n"
#define A_DOT2(i)  "v_dot2_u32_u16 %" #i ", %" #i ", %8, %9\n"
#define A_MIN(i)   "v_min_u32 %" #i ", %" #i ", %8\n"
#define A_LSHLADD(i) "v_lshl_add_u32 %" #i ", %" #i ", 16, %8\n"
#define A_ADD(i) "v_add_u32 %" #i ", %" #i ", %8\n"
#define A_ADD3(i) "v_add3_u32 %" #i ", %" #i ", %8, %9\n"
#define A_MADU16(i) "v_mad_u32_u16 %" #i ", %" #i ", %8, %9\n"
#define A_MULHI(i) "v_mul_hi_u32 %" #i ", %" #i ", %8\n"
#define A_XOR(i) "v_xor_b32 %" #i ", %" #i ", %8\n"
#define A_ALIGNBIT(i) "v_alignbit_b32 %" #i ", %" #i ", %8, 13\n"
#define A_PKMUL16(i) "v_pk_mul_lo_u16 %" #i ", %" #i ", %8\n"
#define A_PKMAD16(i) "v_pk_mad_u16 %" #i ", %" #i ", %8, %9\n"
DEF_KERNEL(k_mullo, A_MULLO)
DEF_KERNEL(k_mad24, A_MAD24)
DEF_KERNEL(k_mul24, A_MUL24)
DEF_KERNEL(k_dot2, A_DOT2)
DEF_KERNEL(k_min, A_MIN)
DEF_KERNEL(k_lshladd, A_LSHLADD)
DEF_KERNEL(k_add, A_ADD)
DEF_KERNEL(k_add3, A_ADD3)
DEF_KERNEL(k_madu16, A_MADU16)
DEF_KERNEL(k_mulhi, A_MULHI)
DEF_KERNEL(k_xor, A_XOR)
DEF_KERNEL(k_alignbit, A_ALIGNBIT)
DEF_KERNEL(k_pkmul16, A_PKMUL16)
DEF_KERNEL(k_pkmad16, A_PKMAD16)

// 64-bit forms
__global__ void k_mad64(uint32_t* out, uint32_t s) {
  uint64_t r0 = threadIdx.x, r1 = r0 + 1, r2 = r0 + 2, r3 = r0 + 3, r4 = r0 + 4, r5 = r0 + 5, r6 = r0 + 6, r7 = r0 + 7;
  uint32_t x = s ^ threadIdx.x, y = s + 77;
  for (int i = 0; i < ITER; ++i) {
#define A_MAD64(i) "v_mad_u64_u32 %" #i ", vcc, %8, %9, %" #i "\n"
    asm volatile(A_MAD64(0) A_MAD64(1) A_MAD64(2) A_MAD64(3) A_MAD64(4) A_MAD64(5) A_MAD64(6) A_MAD64(7)
                 : "+v"(r0), "+v"(r1), "+v"(r2), "+v"(r3), "+v"(r4), "+v"(r5), "+v"(r6), "+v"(r7) : "v"(x), "v"(y) : "vcc");
  }
  uint64_t r = r0 ^ r1 ^ r2 ^ r3 ^ r4 ^ r5 ^ r6 ^ r7;
  out[blockIdx.x * blockDim.x + threadIdx.x] = (uint32_t)r ^ (uint32_t)(r >> 32);
}
__global__ void k_cmp64(uint32_t* out, uint32_t s) {
  uint64_t r0 = threadIdx.x, r1 = r0 + 1, r2 = r0 + 2, r3 = r0 + 3;
  uint64_t x = ((uint64_t)s << 32) ^ threadIdx.x;
  for (int i = 0; i < ITER; ++i) {
#define A_CMP64(i) "v_cmp_lt_u64 vcc, %4, %" #i "\n"
    asm volatile(A_CMP64(0) A_CMP64(1) A_CMP64(2) A_CMP64(3)
                 : "+v"(r0), "+v"(r1), "+v"(r2), "+v"(r3) : "v"(x) : "vcc");
  }
  uint64_t r = r0 ^ r1 ^ r2 ^ r3;
  out[blockIdx.x * blockDim.x + threadIdx.x] = (uint32_t)r ^ (uint32_t)(r >> 32);
}
__global__ void k_lshladd64(uint32_t* out, uint32_t s) {
  uint64_t r0 = threadIdx.x, r1 = r0 + 1, r2 = r0 + 2, r3 = r0 + 3, r4 = r0 + 4, r5 = r0 + 5, r6 = r0 + 6, r7 = r0 + 7;
  uint64_t x = ((uint64_t)s << 32) ^ threadIdx.x;
  for (int i = 0; i < ITER; ++i) {
#define A_LA64(i) "v_lshl_add_u64 %" #i ", %" #i ", 0, %8\n"
    asm volatile(A_LA64(0) A_LA64(1) A_LA64(2) A_LA64(3) A_LA64(4) A_LA64(5) A_LA64(6) A_LA64(7)
                 : "+v"(r0), "+v"(r1), "+v"(r2), "+v"(r3), "+v"(r4), "+v"(r5), "+v"(r6), "+v"(r7) : "v"(x));
  }
  uint64_t r = r0 ^ r1 ^ r2 ^ r3 ^ r4 ^ r5 ^ r6 ^ r7;
  out[blockIdx.x * blockDim.x + threadIdx.x] = (uint32_t)r ^ (uint32_t)(r >> 32);
}

template <typename F>
int run(const char* name, F kern, int insts_per_iter, uint32_t* d_out, int cus, double clk_ghz) {
  int blocks = cus * 8, threads = 256;  // 8 WG x 4 waves per CU = 8 waves per SIMD
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0)); CHECK(hipEventCreate(&e1));
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(threads), 0, 0, d_out, 12345u);
  CHECK(hipDeviceSynchronize());
  CHECK(hipEventRecord(e0));
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(threads), 0, 0, d_out, 12345u);
  CHECK(hipEventRecord(e1));
  CHECK(hipEventSynchronize(e1));
  float ms; CHECK(hipEventElapsedTime(&ms, e0, e1));
  double wave_insts = (double)blocks * (threads / 64) * ITER * insts_per_iter;
  double per_cu_per_cycle = wave_insts / cus / (ms * 1e-3 * clk_ghz * 1e9);
  printf("%-12s %8.3f ms  %6.3f wave-inst/cycle/CU  (=> %5.2f cycles per wave-inst per SIMD)\n", name, ms, per_cu_per_cycle, 4.0 / per_cu_per_cycle);
  return 0;
}
int main() {
  hipDeviceProp_t p; CHECK(hipGetDeviceProperties(&p, 0));
  int cus = p.multiProcessorCount; double clk = p.clockRate / 1e6;
  printf("device %s CUs %d clock %.3f GHz LDS/block %zu L2 %d\n", p.gcnArchName, cus, clk, p.sharedMemPerBlock, p.l2CacheSize);
  uint32_t* d; CHECK(hipMalloc(&d, (size_t)cus * 8 * 256 * 4));
  run("mul_lo_u32", k_mullo, 8, d, cus, clk);
  run("mul_hi_u32", k_mulhi, 8, d, cus, clk);
  run("mad_u64_u32", k_mad64, 8, d, cus, clk);
  run("mad_u32_u24", k_mad24, 8, d, cus, clk);
  run("mul_u32_u24", k_mul24, 8, d, cus, clk);
  run("mad_u32_u16", k_madu16, 8, d, cus, clk);
  run("dot2_u32_u16", k_dot2, 8, d, cus, clk);
  run("pk_mul_lo_u16", k_pkmul16, 8, d, cus, clk);
  run("pk_mad_u16", k_pkmad16, 8, d, cus, clk);
  run("min_u32", k_min, 8, d, cus, clk);
  run("lshl_add_u32", k_lshladd, 8, d, cus, clk);
  run("add_u32", k_add, 8, d, cus, clk);
  run("add3_u32", k_add3, 8, d, cus, clk);
  run("xor_b32", k_xor, 8, d, cus, clk);
  run("alignbit", k_alignbit, 8, d, cus, clk);
  run("cmp_lt_u64", k_cmp64, 4, d, cus, clk);
  run("lshl_add_u64", k_lshladd64, 8, d, cus, clk);
  return 0;
}
