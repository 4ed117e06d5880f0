// Issue rates of the vector instructions that 64-bit modular arithmetic is built from, on gfx950.
//
// Each kernel runs one instruction in eight independent dependency chains per lane (so latency is hidden) for a fixed
// number of iterations on every SIMD of the machine with kWaves waves per SIMD, and the host reports wave-instructions
// per SIMD per cycle from the launch's duration and the shader clock it measures beside it.  1 / (4 cycles) = 0.25 is
// the full rate of a 64-lane wave on a 16-lane SIMD.
//
// Build: make issue_rate (this directory); run: ../issue_rate
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#define HIP_OK(e)                                                                   \
  do {                                                                              \
    hipError_t _e = (e);                                                            \
    if (_e != hipSuccess) {                                                         \
      fprintf(stderr, "%s: %s\n", #e, hipGetErrorString(_e));                       \
      exit(1);                                                                      \
    }                                                                               \
  } while (0)

constexpr int kIters = 2048, kChains = 8, kUnroll = 4;

// One instruction per chain per step; OPS lists the asm text with %0 = chain register (read and written), %1 and %2 =
// loop-invariant operands.
#define CHAIN_KERNEL(NAME, TYPE, CONSTRAINT, ASM, CLOBBER)                                           \
  __global__ __launch_bounds__(256) void NAME(TYPE* out, TYPE a, TYPE b) {                           \
    TYPE c[kChains];                                                                                 \
    for (int k = 0; k < kChains; ++k) c[k] = out[threadIdx.x + 256 * k];                             \
    for (int it = 0; it < kIters / kUnroll; ++it) {                                                  \
      _Pragma("unroll") for (int u = 0; u < kUnroll; ++u) {                                          \
        _Pragma("unroll") for (int k = 0; k < kChains; ++k)                                          \
            asm volatile(ASM : "+" CONSTRAINT(c[k]) : CONSTRAINT(a), CONSTRAINT(b) : CLOBBER);       \
      }                                                                                              \
    }                                                                                                \
    TYPE s = c[0];                                                                                   \
    for (int k = 1; k < kChains; ++k) s += c[k];                                                     \
    out[blockIdx.x * 256 + threadIdx.x] = s;                                                         \
  }

CHAIN_KERNEL(k_add_u32, uint32_t, "v", "v_add_u32 %0, %0, %1", "memory")
CHAIN_KERNEL(k_mul_lo_u32, uint32_t, "v", "v_mul_lo_u32 %0, %0, %1", "memory")
CHAIN_KERNEL(k_mul_hi_u32, uint32_t, "v", "v_mul_hi_u32 %0, %0, %1", "memory")
CHAIN_KERNEL(k_mul_u32_u24, uint32_t, "v", "v_mul_u32_u24 %0, %0, %1", "memory")
CHAIN_KERNEL(k_mad_u32_u24, uint32_t, "v", "v_mad_u32_u24 %0, %0, %1, %2", "memory")
CHAIN_KERNEL(k_cndmask, uint32_t, "v", "v_cndmask_b32 %0, %0, %1, vcc", "memory")
CHAIN_KERNEL(k_fma_f64, double, "v", "v_fma_f64 %0, %0, %1, %2", "memory")
CHAIN_KERNEL(k_mul_f64, double, "v", "v_mul_f64 %0, %0, %1", "memory")
CHAIN_KERNEL(k_add_f64, double, "v", "v_add_f64 %0, %0, %1", "memory")
CHAIN_KERNEL(k_rndne_f64, double, "v", "v_rndne_f64 %0, %0", "memory")
CHAIN_KERNEL(k_lshlrev_b64, uint64_t, "v", "v_lshlrev_b64 %0, 1, %0", "memory")
CHAIN_KERNEL(k_lshrrev_b64, uint64_t, "v", "v_lshrrev_b64 %0, 1, %0", "memory")
CHAIN_KERNEL(k_cmp_u64, uint64_t, "v", "v_cmp_ge_u64 vcc, %0, %1", "vcc")

// v_mad_u64_u32: 32 x 32 + 64 -> 64, the carry goes to vcc
__global__ __launch_bounds__(256) void k_mad_u64_u32(uint64_t* out, uint32_t a, uint32_t b) {
  uint64_t c[kChains];
  uint32_t x[kChains];
  for (int k = 0; k < kChains; ++k) {
    c[k] = out[threadIdx.x + 256 * k];
    x[k] = (uint32_t)c[k] | a;
  }
  for (int it = 0; it < kIters / kUnroll; ++it) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
      for (int k = 0; k < kChains; ++k)
        asm volatile("v_mad_u64_u32 %0, vcc, %1, %2, %0" : "+v"(c[k]) : "v"(x[k]), "v"(b) : "vcc");
    }
  }
  uint64_t s = c[0];
  for (int k = 1; k < kChains; ++k) s += c[k];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}

// v_cvt_f64_u32: 32-bit integer to double
__global__ __launch_bounds__(256) void k_cvt_f64_u32(double* out, uint32_t a, uint32_t b) {
  double c[kChains];
  uint32_t x[kChains];
  for (int k = 0; k < kChains; ++k) {
    c[k] = out[threadIdx.x + 256 * k];
    x[k] = a + k + threadIdx.x;
  }
  for (int it = 0; it < kIters / kUnroll; ++it) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
      for (int k = 0; k < kChains; ++k) asm volatile("v_cvt_f64_u32 %0, %1" : "=v"(c[k]) : "v"(x[k]) : "memory");
    }
  }
  double s = c[0];
  for (int k = 1; k < kChains; ++k) s += c[k];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}

// shader clock: s_memtime counts at a constant 100 MHz on this part, so the clock is taken from a timed loop of
// instructions of known full rate instead (v_add_u32 below)
template <class T, class A>
static double time_kernel(void (*kern)(T*, A, A), T* buf, A a, A b, int blocks, int reps) {
  hipEvent_t e0, e1;
  HIP_OK(hipEventCreate(&e0));
  HIP_OK(hipEventCreate(&e1));
  for (int w = 0; w < 20; ++w) hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), 0, 0, buf, a, b);
  HIP_OK(hipEventRecord(e0, 0));
  for (int r = 0; r < reps; ++r) hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), 0, 0, buf, a, b);
  HIP_OK(hipEventRecord(e1, 0));
  HIP_OK(hipEventSynchronize(e1));
  float ms = 0;
  HIP_OK(hipEventElapsedTime(&ms, e0, e1));
  HIP_OK(hipEventDestroy(e0));
  HIP_OK(hipEventDestroy(e1));
  return ms * 1e-3 / reps;
}

int main() {
  hipDeviceProp_t prop;
  HIP_OK(hipGetDeviceProperties(&prop, 0));
  const int cus = prop.multiProcessorCount, simds = cus * 4;
  const int waves_per_simd = 4;  // 4 waves x 8 chains: 32 independent instructions per SIMD in flight
  const int blocks = cus * waves_per_simd;  // 256 threads = 4 waves, one per SIMD
  const int reps = 20;
  void* buf = nullptr;
  HIP_OK(hipMalloc(&buf, (size_t)blocks * 256 * 8 + 256 * 8 * kChains));
  HIP_OK(hipMemset(buf, 0, (size_t)blocks * 256 * 8 + 256 * 8 * kChains));
  const double instr_per_simd = (double)kIters * kChains * waves_per_simd;
  // The clock during such a loop (no memory traffic) is read from the device's counter
  int clock_khz = 0;
  HIP_OK(hipDeviceGetAttribute(&clock_khz, hipDeviceAttributeClockRate, 0));
  printf("device: %s, %d CUs, %d SIMDs, nominal clock %.0f MHz\n", prop.name, cus, simds, clock_khz / 1e3);
  printf("%-16s %12s %22s %18s\n", "instruction", "us / launch", "wave-instr / SIMD / ns", "relative to add_u32");
  double base = 0;
#define RUN(NAME, T, A, a, b)                                                          \
  do {                                                                                 \
    double s = time_kernel<T, A>(NAME, (T*)buf, (A)(a), (A)(b), blocks, reps);         \
    double rate = instr_per_simd / (s * 1e9);                                          \
    if (base == 0) base = rate;                                                        \
    printf("%-16s %12.1f %22.4f %18.3f\n", &#NAME[2], s * 1e6, rate, rate / base);     \
  } while (0)
  RUN(k_add_u32, uint32_t, uint32_t, 3, 5);
  RUN(k_cndmask, uint32_t, uint32_t, 3, 5);
  RUN(k_mul_u32_u24, uint32_t, uint32_t, 3, 5);
  RUN(k_mad_u32_u24, uint32_t, uint32_t, 3, 5);
  RUN(k_mul_lo_u32, uint32_t, uint32_t, 3, 5);
  RUN(k_mul_hi_u32, uint32_t, uint32_t, 3, 5);
  RUN(k_mad_u64_u32, uint64_t, uint32_t, 3, 5);
  RUN(k_lshlrev_b64, uint64_t, uint64_t, 3, 5);
  RUN(k_lshrrev_b64, uint64_t, uint64_t, 3, 5);
  RUN(k_cmp_u64, uint64_t, uint64_t, 3, 5);
  RUN(k_add_f64, double, double, 1.0000001, 0.5);
  RUN(k_mul_f64, double, double, 1.0000001, 0.5);
  RUN(k_fma_f64, double, double, 1.0000001, 0.5);
  RUN(k_rndne_f64, double, double, 1.0000001, 0.5);
  RUN(k_cvt_f64_u32, double, uint32_t, 3, 5);
  HIP_OK(hipFree(buf));
  return 0;
}
