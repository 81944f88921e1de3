// Measuring instrument, not part of the library: times the headline kernel (gemm_m16_kernel, bf16,
// 8192 x 8192 x 8192 by default) with parts of its main loop taken out, to attribute time and -- under
// the power limit, through the clock the device sustains -- energy to them.  Compiled once per variant:
//   -DSRT_ABLATE=<bits>   see gemm_mfma_m16.h (1 no barrier, 2 no operand traffic, 4 fragments stay in
//                         registers, 8 every workgroup requests tile 0)
//   -DABL_NS=<3|4|5>      ring depth (prefetch distance NS - 1 stages)
//   -DABL_DEEP=1          the 64-deep form of the kernel (gemm_mfma_m16d.h; no ablation switches)
//   -DABL_TAIL=1          (with ABL_DEEP) the tail-sharing form; every element of its result is then compared
//                         with the plain 64-deep kernel's
//   -DABL_AKC / -DABL_BKC operand layouts (defaults 1 / 0: the headline's row-major A and B)
// Run: ablate_m16 [normal|zero] [M N K [pad]]; pad: elements added to the pitch of the operands' rows; operands ~ N(0,1)/sqrt(K) (generated on the device) or zeros.
// Prints one line: variant, data, median and minimum time per launch, TFLOP/s, and (unablated builds) the
// largest error of 64 sampled results against a double-precision dot product.
#define SRT_M16_ANY_RING_DEPTH 1
#include "gemm_mfma_m16d.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#ifndef ABL_NS
#define ABL_NS 5
#endif
#ifndef ABL_DEEP
#define ABL_DEEP 0
#endif
#ifndef ABL_TAIL
#define ABL_TAIL 0
#endif
#ifndef ABL_AKC
#define ABL_AKC 1
#endif
#ifndef ABL_BKC
#define ABL_BKC 0
#endif

#define CHECK(x)                                                              \
  do {                                                                        \
    hipError_t e_ = (x);                                                      \
    if (e_ != hipSuccess) {                                                   \
      fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                 \
      exit(1);                                                                \
    }                                                                         \
  } while (0)

namespace {

__device__ inline uint32_t mix(uint32_t x) {
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}

__global__ void fill_normal(uint16_t* dst, size_t n, float scale, uint32_t seed, int zero) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    float v = 0.0f;
    if (!zero) {
      const uint32_t s = seed + (uint32_t)i * 2u;
      const float u1 = (mix(s) >> 8) * (1.0f / 16777216.0f) + 1e-7f;
      const float u2 = (mix(s + 1u) >> 8) * (1.0f / 16777216.0f);
      v = sqrtf(-2.0f * logf(u1)) * cosf(6.2831853f * u2) * scale;
    }
    dst[i] = srt::BF16::from_float(v);
  }
}

float bf16_to_float(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

}  // namespace

// The tail-sharing launcher takes its workspace from the library's allocator; this probe stands alone.
extern "C" srtStatus srtDeviceAllocate(void** ptr, size_t size, srtStream) {
  static void* block = nullptr;
  static size_t held = 0;
  if (size > held) {
    if (block) (void)hipFree(block);
    if (hipMalloc(&block, size) != hipSuccess) return srtErrorOutOfMemory;
    held = size;
  }
  *ptr = block;
  return srtSuccess;
}
extern "C" srtStatus srtDeviceFree(void*) { return srtSuccess; }

int main(int argc, char** argv) {
  const bool zero = argc > 1 && strcmp(argv[1], "zero") == 0;
  int M = 8192, N = 8192, K = 8192;
  if (argc > 4) { M = atoi(argv[2]); N = atoi(argv[3]); K = atoi(argv[4]); }
  const int pad = argc > 5 ? atoi(argv[5]) : 0;   // elements added to the pitch of every operand row (a multiple of 8)
  if (M % 256 || N % 256 || K % 32 || K < 160) { fprintf(stderr, "M, N multiples of 256; K a multiple of 32, at least 160\n"); return 1; }
  uint16_t *a, *b, *c;
  // pitches of the stored rows: A is [M][K] or [K][M], B is [N][K] or [K][N]
  const size_t a_rows = ABL_AKC ? M : K, a_pitch = (ABL_AKC ? K : M) + pad;
  const size_t b_rows = ABL_BKC ? N : K, b_pitch = (ABL_BKC ? K : N) + pad;
  CHECK(hipMalloc(&a, a_rows * a_pitch * 2));
  CHECK(hipMalloc(&b, b_rows * b_pitch * 2));
  CHECK(hipMalloc(&c, (size_t)M * N * 2));
  const float scale = 1.0f / sqrtf((float)K);
  hipLaunchKernelGGL(fill_normal, dim3(4096), dim3(256), 0, 0, a, a_rows * a_pitch, scale, 0x1234567u, zero ? 1 : 0);
  hipLaunchKernelGGL(fill_normal, dim3(4096), dim3(256), 0, 0, b, b_rows * b_pitch, scale, 0x89abcdeu, zero ? 1 : 0);
  CHECK(hipDeviceSynchronize());

  srt::GemmProblem p{};
  p.dtype = srtReal16BF;
  p.M = M; p.N = N; p.K = K; p.batch = 1;
  p.A = a; p.B = b; p.C = c;
  // A stored [M, K] (k-contiguous) or [K, M]; B stored [N, K] (k-contiguous) or [K, N]
  if (ABL_AKC) { p.sam = (long long)a_pitch; p.sak = 1; } else { p.sam = 1; p.sak = (long long)a_pitch; }
  if (ABL_BKC) { p.sbn = (long long)b_pitch; p.sbk = 1; } else { p.sbn = 1; p.sbk = (long long)b_pitch; }
  p.scm = N; p.scn = 1;
  p.activation = srtActivationIdentity;

  auto launch = [&]() {
    if (ABL_DEEP && ABL_TAIL) CHECK((srt::m16d::launch_tail_kernel<srt::BF16, ABL_AKC != 0, ABL_BKC != 0, srt::m16::EPI_PLAIN>(p, 0)));
    else if (ABL_DEEP) CHECK((srt::m16d::launch_kernel<srt::BF16, ABL_AKC != 0, ABL_BKC != 0, srt::m16::EPI_PLAIN>(p, 0)));
    else CHECK((srt::m16::launch_kernel<srt::BF16, ABL_AKC != 0, ABL_BKC != 0, srt::m16::EPI_PLAIN, ABL_NS, 8>(p, 0)));
  };
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  auto group_ms = [&](int launches) {
    CHECK(hipEventRecord(e0));
    for (int i = 0; i < launches; ++i) launch();
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    return ms / launches;
  };
  const double flop = 2.0 * M * N * K;
  const int per_group = std::max(4, (int)(20.0 * 1.1e12 / flop));
  // settle: at least 0.6 s of load
  double spent = 0.0;
  while (spent < 600.0) spent += group_ms(per_group) * per_group;
  std::vector<float> t;
  for (int g = 0; g < 7; ++g) t.push_back(group_ms(per_group));
  std::sort(t.begin(), t.end());
  const float med = t[t.size() / 2];

  double worst = -1.0;
  if (SRT_ABLATE == 0 && !zero) {
    // 64 sampled results against double-precision dot products of the stored operands
    std::vector<uint16_t> ha(a_rows * a_pitch), hb(b_rows * b_pitch), hc((size_t)M * N);
    CHECK(hipMemcpy(ha.data(), a, ha.size() * 2, hipMemcpyDeviceToHost));
    CHECK(hipMemcpy(hb.data(), b, hb.size() * 2, hipMemcpyDeviceToHost));
    CHECK(hipMemcpy(hc.data(), c, hc.size() * 2, hipMemcpyDeviceToHost));
    worst = 0.0;
    for (int s = 0; s < 64; ++s) {
      const int m = (int)(((long long)s * 2654435761LL) % M), n = (int)(((long long)s * 40503LL * 977) % N);
      double ref = 0.0;
      for (int k = 0; k < K; ++k)
        ref += (double)bf16_to_float(ha[(size_t)m * p.sam + (size_t)k * p.sak]) *
               (double)bf16_to_float(hb[(size_t)k * p.sbk + (size_t)n * p.sbn]);
      worst = std::max(worst, fabs(ref - (double)bf16_to_float(hc[(size_t)m * N + n])));
    }
  }
  long long differing = -1;
  double worst_pair = 0.0;
  if (ABL_DEEP && ABL_TAIL && !zero) {
    std::vector<uint16_t> tail((size_t)M * N), plain((size_t)M * N);
    CHECK(hipMemcpy(tail.data(), c, tail.size() * 2, hipMemcpyDeviceToHost));
    CHECK((srt::m16d::launch_kernel<srt::BF16, ABL_AKC != 0, ABL_BKC != 0, srt::m16::EPI_PLAIN>(p, 0)));
    CHECK(hipDeviceSynchronize());
    CHECK(hipMemcpy(plain.data(), c, plain.size() * 2, hipMemcpyDeviceToHost));
    differing = 0;
    for (size_t i = 0; i < tail.size(); ++i) {
      if (tail[i] != plain[i]) ++differing;
      worst_pair = std::max(worst_pair, (double)fabsf(bf16_to_float(tail[i]) - bf16_to_float(plain[i])));
    }
  }
#ifdef SRT_TAIL_TRACE
  if (ABL_DEEP) {
    // one more launch, then the piece boundaries of some workgroups relative to the earliest start, in us
    std::vector<unsigned long long> tr(256 * 16, 0);
    CHECK(hipMemcpyToSymbol(HIP_SYMBOL(srt::m16d::tail_trace), tr.data(), tr.size() * 8));
    launch();
    CHECK(hipDeviceSynchronize());
    CHECK(hipMemcpyFromSymbol(tr.data(), HIP_SYMBOL(srt::m16d::tail_trace), tr.size() * 8));
    unsigned long long t0 = ~0ull;
    for (int w = 0; w < 256; ++w) if (tr[w * 16]) t0 = std::min(t0, tr[w * 16]);
    for (int w = 0; w < 256; w += (w < 4 ? 1 : 21)) {
      printf("wg %3d:", w);
      for (int e = 0; e < 16 && tr[w * 16 + e]; ++e) printf(" %.1f", (double)(tr[w * 16 + e] - t0) / 100.0);
      printf("\n");
    }
  }
#endif
  printf("ablate=%d deep=%d ns=%d akc=%d bkc=%d %-6s M=%d N=%d K=%d: median %.4f ms %.1f TFLOP/s (min %.4f ms %.1f)", SRT_ABLATE,
         ABL_DEEP + 10 * ABL_TAIL, ABL_NS, ABL_AKC, ABL_BKC, zero ? "zero" : "normal", M, N, K, med, flop / (med * 1e-3) * 1e-12, t[0],
         flop / (t[0] * 1e-3) * 1e-12);
  if (worst >= 0.0) printf("  max |error| of 64 samples %.3g (|c| ~ %.2g)", worst, 1.0 / sqrt((double)K) * sqrt((double)K) / sqrt((double)K));
  if (differing >= 0) printf("  vs plain kernel: %lld of %lld elements differ, largest difference %.3g", differing, (long long)M * N, worst_pair);
  printf("\n");
  return 0;
}
