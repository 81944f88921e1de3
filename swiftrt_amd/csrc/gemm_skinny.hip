// Small-M matmul (M <= 32) against a k-contiguous weight: out[m, n] = sum_k x[m, k] * W[n, k].
// The shape of single-token / small-batch inference; bound by streaming W from HBM once.
//
// No LDS staging and no barrier in the k loop: the MFMA B-operand layout (lane l holds 8
// consecutive k of column l % 32) is exactly a 16-byte global load of row n of W, so each lane
// loads its operand straight from memory.  The order of k inside one MFMA is free as long as
// both operands agree, so lane (n, h) reads the 64 contiguous bytes k0 + 32 h .. k0 + 32 h + 31
// (four 16-byte loads, one per MFMA step) and a wave consumes whole 128-byte lines of each row.
//   block   4 waves share 32 rows of W (one 32 x 32 output tile, rows m >= M are zero);
//           wave w takes the 64-wide k blocks w, w + 4, ...; partial tiles are summed through
//           LDS once at the end, then bias + activation + store.
//   grid    ceil(N / 32) x batch workgroups, all resident at once: the HBM pipe sees
//           every row's stream concurrently.
#include "gemm_common.h"

namespace srt {

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

template <typename T>
__device__ __forceinline__ f32x16_t mfma32s(u32x4_t a, u32x4_t b, f32x16_t c);
template <>
__device__ __forceinline__ f32x16_t mfma32s<BF16>(u32x4_t a, u32x4_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b),
                                                 c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x16_t mfma32s<F16>(u32x4_t a, u32x4_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b),
                                                c, 0, 0, 0);
}

constexpr int SK_WAVES = 4;
constexpr int SK_KB = 64;  // k per block step

struct Frag4 {
  u32x4_t c[4];
};

// four 16-byte chunks at row_ptr + k0 + 32 h + 8 s, zero beyond K
__device__ __forceinline__ void load_frag(Frag4& f, const uint16_t* row_ptr, int k0, int h, int K, bool row_ok) {
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const int k = k0 + 32 * h + 8 * s;
    u32x4_t x = {0u, 0u, 0u, 0u};
    if (row_ok && k < K) x = *reinterpret_cast<const u32x4_t*>(row_ptr + k);
    f.c[s] = x;
  }
}

template <typename T>
__global__ __launch_bounds__(SK_WAVES * 64) void gemm_skinny_kernel(GemmProblem p) {
  __shared__ float red[SK_WAVES][16][64];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, h = lane >> 5;
  const int n0 = blockIdx.x * 32;
  const int bz = blockIdx.y;

  const uint16_t* X = (const uint16_t*)p.A + (long long)bz * p.sab;
  const uint16_t* W = (const uint16_t*)p.B + (long long)bz * p.sbb;

  const int n = n0 + r;
  const bool n_ok = n < p.N;
  const bool m_ok = r < p.M;
  const uint16_t* wrow = W + (long long)(n_ok ? n : 0) * p.sbn;
  const uint16_t* xrow = X + (long long)(m_ok ? r : 0) * p.sam;

  f32x16_t acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.0f;

  const int KB = (p.K + SK_KB - 1) / SK_KB;
  Frag4 w0, x0, w1, x1;
  int kb = wave;
  if (kb < KB) {
    load_frag(w0, wrow, kb * SK_KB, h, p.K, n_ok);
    load_frag(x0, xrow, kb * SK_KB, h, p.K, m_ok);
  }
  // two k blocks per trip: loads for the next pair are in flight while this pair multiplies
  for (; kb < KB; kb += 2 * SK_WAVES) {
    const int kb1 = kb + SK_WAVES;
    const bool has1 = kb1 < KB;
    if (has1) {
      load_frag(w1, wrow, kb1 * SK_KB, h, p.K, n_ok);
      load_frag(x1, xrow, kb1 * SK_KB, h, p.K, m_ok);
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) acc = mfma32s<T>(x0.c[s], w0.c[s], acc);
    const int kb2 = kb1 + SK_WAVES;
    if (kb2 < KB) {
      load_frag(w0, wrow, kb2 * SK_KB, h, p.K, n_ok);
      load_frag(x0, xrow, kb2 * SK_KB, h, p.K, m_ok);
    }
    if (has1) {
#pragma unroll
      for (int s = 0; s < 4; ++s) acc = mfma32s<T>(x1.c[s], w1.c[s], acc);
    }
  }

#pragma unroll
  for (int v = 0; v < 16; ++v) red[wave][v][lane] = acc[v];
  __syncthreads();

  // wave w finishes accumulator registers 4w .. 4w+3: rows m = 8 w + 4 h + i, column n
  if (!n_ok) return;
  Epilogue<T> ep(p);
  uint16_t* C = (uint16_t*)p.C + (long long)bz * p.scb;
  const float bcol = ep.per_row ? 0.0f : ep.bias_at(0, n);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int v = 4 * wave + i;
    const int m = 8 * wave + 4 * h + i;
    if (m >= p.M) continue;
    float s = 0.0f;
#pragma unroll
    for (int w = 0; w < SK_WAVES; ++w) s += red[w][v][lane];
    const float bv = ep.per_row ? ep.bias_at(m, n) : bcol;
    C[(long long)m * p.scm + (long long)n * p.scn] = ep.finish(s, bv);
  }
}

inline bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

}  // namespace

bool skinny_supported(const GemmProblem& p) {
  if (p.dtype != srtReal16BF && p.dtype != srtReal16F) return false;
  if (p.M > 32 || p.M < 1 || p.K < 1) return false;
  if (p.sak != 1 || p.sbk != 1) return false;           // both operands k-contiguous
  if ((p.K % 8) != 0) return false;                     // whole 16-byte chunks
  if ((p.sam % 8) != 0 && p.M > 1) return false;
  if ((p.sbn % 8) != 0 && p.N > 1) return false;
  if ((p.sab % 8) != 0 || (p.sbb % 8) != 0) return false;
  if (p.sam < 0 || p.sbn < 0 || p.scm < 0 || p.scn < 0) return false;
  if (!aligned16(p.A) || !aligned16(p.B)) return false;
  if (p.batch > 65535) return false;
  // worth it only when the weight dominates the traffic
  return p.N >= 32;
}

hipError_t launch_skinny(const GemmProblem& p, hipStream_t stream) {
  dim3 grid((p.N + 31) / 32, p.batch);
  dim3 block(SK_WAVES * 64);
  if (p.dtype == srtReal16BF) hipLaunchKernelGGL(gemm_skinny_kernel<BF16>, grid, block, 0, stream, p);
  else hipLaunchKernelGGL(gemm_skinny_kernel<F16>, grid, block, 0, stream, p);
  return hipGetLastError();
}

}  // namespace srt
