// Measures what the matrix cores of this device sustain on a loop of nothing but
// v_mfma_f32_16x16x32_bf16 -- the instruction of the headline GEMM kernel, and the cheaper per flop
// of the two bf16 shapes -- with operands held in registers and the accumulator set of a
// 128 x 128 wave tile (8 x 8 tiles, all 256 accumulator registers): no memory traffic, no LDS,
// every SIMD of every CU busy.  Run once with operands drawn from N(0,1)/sqrt(8192) -- the distribution of the
// benchmark's GEMM inputs -- and once with all-zero operands.  The part lowers its clock under
// the power the first case draws, so the first figure, not the data-sheet peak, is what any GEMM
// kernel on real data can approach on this device; the second shows the clock is back at its
// maximum when the multipliers do not toggle.  The shader clock is read in-kernel (cycle counter
// against the constant 100 MHz counter).
//
// Prints one JSON object.  A stand-alone program: it is a measuring instrument for bench.py, not
// part of the library.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

#define CHECK(x)                                                                  \
  do {                                                                            \
    hipError_t e_ = (x);                                                          \
    if (e_ != hipSuccess) {                                                       \
      fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                     \
      exit(1);                                                                    \
    }                                                                             \
  } while (0)

namespace {

constexpr int OPERANDS = 8;          // A and B fragments of one k step of the wave tile
constexpr int MFMA_PER_ITER = OPERANDS * OPERANDS;

__device__ inline uint32_t mix(uint32_t x) {
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}
__device__ inline float normal(uint32_t s) {
  const float u1 = (mix(s) >> 8) * (1.0f / 16777216.0f) + 1e-7f;
  const float u2 = (mix(s ^ 0x9e3779b9u) >> 8) * (1.0f / 16777216.0f);
  return sqrtf(-2.0f * logf(u1)) * cosf(6.2831853f * u2);
}

__global__ __launch_bounds__(256) void mfma_loop(int iters, int real_data, float* sink, long long* clocks) {
  bf16x8_t a[OPERANDS], b[OPERANDS];
  const uint32_t seed = (blockIdx.x * 256 + threadIdx.x) * 256;
  for (int i = 0; i < OPERANDS; ++i)
    for (int j = 0; j < 8; ++j) {
      a[i][j] = (__bf16)(real_data ? normal(seed + i * 16 + j) * 0.011048543f : 0.0f);
      b[i][j] = (__bf16)(real_data ? normal(seed + i * 16 + j + 8) * 0.011048543f : 0.0f);
    }
  // every definition and use of an accumulator tile inside the timed region is an MFMA with the tile
  // in accumulator registers: the first one of each tile takes the constant 0 as its addend
  f32x4_t acc[OPERANDS][OPERANDS];
#pragma unroll
  for (int j = 0; j < OPERANDS; ++j)
#pragma unroll
    for (int i = 0; i < OPERANDS; ++i)
      asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=a"(acc[i][j]) : "v"(b[j]), "v"(a[i]));
  const long long c0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < OPERANDS; ++j)
#pragma unroll
      for (int i = 0; i < OPERANDS; ++i)
        // written out with the accumulator tied in place: given the builtin, the register allocator
        // rotates the 64 tiles through spare registers with copies between the MFMAs
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(b[j]), "v"(a[i]));
  }
  asm volatile("s_nop 7\n\ts_nop 7" ::: "memory");   // wait states before the accumulators are read
  const long long c1 = clock64(), w1 = wall_clock64();
  float s = 0.0f;
  for (int i = 0; i < OPERANDS; ++i)
    for (int j = 0; j < OPERANDS; ++j)
      for (int v = 0; v < 4; ++v) s += acc[i][j][v];
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    clocks[0] = c1 - c0;
    clocks[1] = w1 - w0;
  }
  if (s == 12345.678f) sink[0] = s;   // keeps the loop alive
}

struct Result { double tflops, ghz; };

Result measure(int cus, int real_data, float* sink, long long* clocks) {
  const int iters = 12000;   // ~ 6 ms per launch
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  Result best{0.0, 0.0};
  for (int rep = 0; rep < 4; ++rep) {   // the first launches run before the clock has settled
    CHECK(hipEventRecord(e0));
    hipLaunchKernelGGL(mfma_loop, dim3(cus), dim3(256), 0, 0, iters, real_data, sink, clocks);
    CHECK(hipGetLastError());
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    long long h[2];
    CHECK(hipMemcpy(h, clocks, sizeof(h), hipMemcpyDeviceToHost));
    const double flop = (double)cus * 4 * iters * MFMA_PER_ITER * (2.0 * 16 * 16 * 32);
    if (rep == 3) best = Result{flop / ms * 1e-9, (double)h[0] / (double)h[1] * 0.1};
  }
  CHECK(hipEventDestroy(e0));
  CHECK(hipEventDestroy(e1));
  return best;
}

}  // namespace

int main() {
  hipDeviceProp_t prop;
  CHECK(hipGetDeviceProperties(&prop, 0));
  float* sink;
  long long* clocks;
  CHECK(hipMalloc(&sink, 64));
  CHECK(hipMalloc(&clocks, 64));
  const int cus = prop.multiProcessorCount;
  const Result zero = measure(cus, 0, sink, clocks);
  const Result real = measure(cus, 1, sink, clocks);
  printf("{\"instruction\": \"v_mfma_f32_16x16x32_bf16\", \"cus\": %d, "
         "\"normal_operands\": {\"tflops\": %.1f, \"clock_ghz\": %.3f}, "
         "\"zero_operands\": {\"tflops\": %.1f, \"clock_ghz\": %.3f}}\n",
         cus, real.tflops, real.ghz, zero.tflops, zero.ghz);
  CHECK(hipFree(sink));
  CHECK(hipFree(clocks));
  return 0;
}
