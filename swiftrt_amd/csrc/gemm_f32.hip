// fp32 matmul on the matrix cores: v_mfma_f32_32x32x2_f32 (true fp32 products and sums, no
// reduced-precision path), any strides.
//
//   tile    64 x 64 x 16 per workgroup of 4 waves (2 x 2, each one 32 x 32 MFMA tile = 16 fp32
//           accumulators per lane); operands are staged through LDS k-major ([k][m], [k][n]) so
//           the MFMA operand of lane l (row / column l % 32, k = 2 kk + l / 32) is one
//           conflict-free ds_read_b32.
//   loads   element-wise with the caller's strides (views, transposes, column-major all land
//           here), next k tile prefetched into registers while the current one multiplies.
//   split   when the 64 x 64 tiles alone would leave most CUs idle (e.g. 512^3 = 64 tiles), the
//           tile shrinks to 32 x 32 and the 4 waves split K between them, summing through LDS.
#include "gemm_common.h"

namespace srt {

namespace {

typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int FT = 64;   // tile edge
constexpr int FK = 16;   // k per stage

// ---- 64 x 64 tiles, waves 2 x 2 ----------------------------------------------------------------
__global__ __launch_bounds__(256) void gemm_f32_mfma_kernel(GemmProblem p) {
  __shared__ float As[2][FK][FT + 4];
  __shared__ float Bs[2][FK][FT + 4];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
  const int r = lane & 31, kh = lane >> 5;
  const int m0 = blockIdx.y * FT, n0 = blockIdx.x * FT, bz = blockIdx.z;
  const float* A = (const float*)p.A + (long long)bz * p.sab;
  const float* B = (const float*)p.B + (long long)bz * p.sbb;
  float* C = (float*)p.C + (long long)bz * p.scb;

  // thread -> element mapping that walks the unit stride first
  const bool a_k_fast = (p.sak == 1), b_n_fast = (p.sbn == 1);
  int am[4], ak[4], bn[4], bk[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = tid + i * 256;
    if (a_k_fast) { ak[i] = idx & (FK - 1); am[i] = idx >> 4; } else { am[i] = idx & (FT - 1); ak[i] = idx >> 6; }
    if (b_n_fast) { bn[i] = idx & (FT - 1); bk[i] = idx >> 6; } else { bk[i] = idx & (FK - 1); bn[i] = idx >> 4; }
  }
  auto fetch = [&](int k0, float (&ra)[4], float (&rb)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + am[i], ka = k0 + ak[i], n = n0 + bn[i], kb = k0 + bk[i];
      ra[i] = (m < p.M && ka < p.K) ? A[(long long)m * p.sam + (long long)ka * p.sak] : 0.0f;
      rb[i] = (n < p.N && kb < p.K) ? B[(long long)kb * p.sbk + (long long)n * p.sbn] : 0.0f;
    }
  };
  auto stash = [&](int buf, const float (&ra)[4], const float (&rb)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      As[buf][ak[i]][am[i]] = ra[i];
      Bs[buf][bk[i]][bn[i]] = rb[i];
    }
  };

  f32x16_t acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.0f;

  float ra[4], rb[4];
  fetch(0, ra, rb);
  stash(0, ra, rb);
  __syncthreads();
  const int KT = (p.K + FK - 1) / FK;
  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT) fetch((kt + 1) * FK, ra, rb);
#pragma unroll
    for (int kk = 0; kk < FK / 2; ++kk)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(As[buf][2 * kk + kh][wm + r], Bs[buf][2 * kk + kh][wn + r], acc, 0, 0, 0);
    if (kt + 1 < KT) stash(buf ^ 1, ra, rb);
    __syncthreads();
  }

  // lane holds column r and rows 8 (v / 4) + 4 kh + v % 4 of the wave's 32 x 32 tile
  Epilogue<F32> ep(p);
  const int n = n0 + wn + r;
  if (n >= p.N) return;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int m = m0 + wm + 8 * (v >> 2) + 4 * kh + (v & 3);
    if (m < p.M) C[(long long)m * p.scm + (long long)n * p.scn] = ep.finish(acc[v], ep.bias_at(m, n));
  }
}

// ---- 32 x 32 tiles, the 4 waves split K ---------------------------------------------------------
// Wave w owns the k tiles w, w + 4, ...; each wave stages its own 32 x 16 / 16 x 32 operand slabs
// in a private LDS area (no workgroup barrier in the k loop); the partial tiles meet in LDS.
__global__ __launch_bounds__(256) void gemm_f32_mfma_splitk_kernel(GemmProblem p) {
  __shared__ float As[4][FK][32 + 1];
  __shared__ float Bs[4][FK][32 + 1];
  __shared__ float red[4][16][64];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, kh = lane >> 5;
  const int m0 = blockIdx.y * 32, n0 = blockIdx.x * 32, bz = blockIdx.z;
  const float* A = (const float*)p.A + (long long)bz * p.sab;
  const float* B = (const float*)p.B + (long long)bz * p.sbb;
  float* C = (float*)p.C + (long long)bz * p.scb;

  const bool a_k_fast = (p.sak == 1), b_n_fast = (p.sbn == 1);
  int am[8], ak[8], bn[8], bk[8];   // a wave fetches 512 + 512 elements per k tile: 8 + 8 per lane
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int idx = lane + i * 64;
    if (a_k_fast) { ak[i] = idx & (FK - 1); am[i] = idx >> 4; } else { am[i] = idx & 31; ak[i] = idx >> 5; }
    if (b_n_fast) { bn[i] = idx & 31; bk[i] = idx >> 5; } else { bk[i] = idx & (FK - 1); bn[i] = idx >> 4; }
  }

  f32x16_t acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.0f;

  const int KT = (p.K + FK - 1) / FK;
  float ra[8], rb[8];
  auto fetch = [&](int kt) {
    const int k0 = kt * FK;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int m = m0 + am[i], ka = k0 + ak[i], n = n0 + bn[i], kb = k0 + bk[i];
      ra[i] = (kt < KT && m < p.M && ka < p.K) ? A[(long long)m * p.sam + (long long)ka * p.sak] : 0.0f;
      rb[i] = (kt < KT && n < p.N && kb < p.K) ? B[(long long)kb * p.sbk + (long long)n * p.sbn] : 0.0f;
    }
  };
  fetch(wave);
  for (int kt = wave; kt < KT; kt += 4) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      As[wave][ak[i]][am[i]] = ra[i];
      Bs[wave][bk[i]][bn[i]] = rb[i];
    }
    fetch(kt + 4);   // next slab in flight while this one multiplies
    // the slab was written and is read by this wave only: LDS operations of one wave execute in
    // order, so no workgroup barrier is needed -- only a wave-level fence that keeps the
    // compiler from moving LDS accesses across it
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int kk = 0; kk < FK / 2; ++kk)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(As[wave][2 * kk + kh][r], Bs[wave][2 * kk + kh][r], acc, 0, 0, 0);
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }

#pragma unroll
  for (int v = 0; v < 16; ++v) red[wave][v][lane] = acc[v];
  __syncthreads();

  // wave w finishes accumulator registers 4 w .. 4 w + 3: rows 8 w + 4 kh + i, column r
  Epilogue<F32> ep(p);
  const int n = n0 + r;
  if (n >= p.N) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int v = 4 * wave + i;
    const int m = m0 + 8 * wave + 4 * kh + i;
    if (m >= p.M) continue;
    const float s = (red[0][v][lane] + red[1][v][lane]) + (red[2][v][lane] + red[3][v][lane]);
    C[(long long)m * p.scm + (long long)n * p.scn] = ep.finish(s, ep.bias_at(m, n));
  }
}

// ---- 32 x 32 tiles, the 4 waves split K; row-major operands, whole k range in flight ------------
// The variant above keeps one 16-deep slab in flight per wave, so a launch-latency-sized problem
// (512^3: 8 slabs per wave) pays one memory round trip per slab.  When both operands are row-major
// with 16-byte aligned rows (A k-contiguous, B n-contiguous) a wave instead requests up to
// SV_SLABS slabs of its k range at once with 16-byte loads (4 per slab and lane), and multiplies
// them as they arrive; wave w owns a contiguous quarter of K.
//   A slab  32 rows x 16 k: lane f (two per lane) loads 4 k of row f / 4; transposed into LDS
//           k-major [k][m], pitch 36: the four ds_write_b32 of a lane pair are conflict-free.
//   B slab  16 k x 32 n: lane f loads 4 n of k row f / 8; LDS [k][n], pitch 32: even k rows sit
//           in banks 0-31 and odd ones in 32-63, which is exactly the split of the MFMA operand
//           read (lanes 0-31 take k = 2 kk, lanes 32-63 k = 2 kk + 1).
constexpr int SV_SLABS = 8;
typedef float f32x4v_t __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void gemm_f32_mfma_splitk_vec_kernel(GemmProblem p) {
  __shared__ float As[4][2][FK][36];
  __shared__ __attribute__((aligned(16))) float Bs[4][2][FK][32];
  __shared__ float red[4][16][64];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, kh = lane >> 5;
  const int m0 = blockIdx.y * 32, n0 = blockIdx.x * 32, bz = blockIdx.z;
  const float* A = (const float*)p.A + (long long)bz * p.sab;
  const float* B = (const float*)p.B + (long long)bz * p.sbb;
  float* C = (float*)p.C + (long long)bz * p.scb;

  // this wave's slabs: a contiguous quarter of the k range
  const int slabs = (p.K + FK - 1) / FK;
  const int per_wave = (slabs + 3) / 4;
  const int first = wave * per_wave;
  const int last = min(slabs, first + per_wave);   // exclusive

  // lane -> 16-byte piece of a slab (two pieces per operand)
  int am[2], ak[2], bk[2], bn[2];
  const float* ap[2];
  const float* bp[2];
  bool a_row_ok[2], b_col_ok[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int f = lane + 64 * i;
    am[i] = f >> 2; ak[i] = (f & 3) * 4;
    bk[i] = f >> 3; bn[i] = (f & 7) * 4;
    a_row_ok[i] = m0 + am[i] < p.M;
    b_col_ok[i] = n0 + bn[i] < p.N;   // N is a multiple of 4: the piece is whole
    ap[i] = A + (long long)(m0 + am[i]) * p.sam + ak[i];
    bp[i] = B + (long long)bk[i] * p.sbk + n0 + bn[i];
  }

  f32x16_t acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.0f;

  for (int s0 = first; s0 < last; s0 += SV_SLABS) {
    f32x4v_t ra[SV_SLABS][2], rb[SV_SLABS][2];
#pragma unroll
    for (int s = 0; s < SV_SLABS; ++s) {
      const int k0 = (s0 + s) * FK;
      const bool live = s0 + s < last;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const f32x4v_t zero = {0.0f, 0.0f, 0.0f, 0.0f};
        // K is a multiple of 4: a piece lies wholly inside or outside the k range
        ra[s][i] = (live && a_row_ok[i] && k0 + ak[i] < p.K) ? *reinterpret_cast<const f32x4v_t*>(ap[i] + k0) : zero;
        rb[s][i] = (live && b_col_ok[i] && k0 + bk[i] < p.K)
                       ? *reinterpret_cast<const f32x4v_t*>(bp[i] + (long long)k0 * p.sbk) : zero;
      }
    }
#pragma unroll
    for (int s = 0; s < SV_SLABS; ++s) {
      if (s0 + s >= last) break;
      const int buf = s & 1;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int e = 0; e < 4; ++e) As[wave][buf][ak[i] + e][am[i]] = ra[s][i][e];
        *reinterpret_cast<f32x4v_t*>(&Bs[wave][buf][bk[i]][bn[i]]) = rb[s][i];
      }
      // the slab is written and read by this wave only: LDS operations of one wave execute in
      // order, so a wave-level fence (for the compiler) is all that is needed; the other buffer
      // may still be read by the MFMAs issued for the previous slab
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int kk = 0; kk < FK / 2; ++kk)
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(As[wave][buf][2 * kk + kh][r], Bs[wave][buf][2 * kk + kh][r], acc, 0, 0, 0);
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
  }

#pragma unroll
  for (int v = 0; v < 16; ++v) red[wave][v][lane] = acc[v];
  __syncthreads();

  // wave w finishes accumulator registers 4 w .. 4 w + 3: rows 8 w + 4 kh + i, column r
  Epilogue<F32> ep(p);
  const int n = n0 + r;
  if (n >= p.N) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int v = 4 * wave + i;
    const int m = m0 + 8 * wave + 4 * kh + i;
    if (m >= p.M) continue;
    const float s = (red[0][v][lane] + red[1][v][lane]) + (red[2][v][lane] + red[3][v][lane]);
    C[(long long)m * p.scm + (long long)n * p.scn] = ep.finish(s, ep.bias_at(m, n));
  }
}

// Preconditions of the vector variant: both operands row-major with 16-byte aligned rows.
bool splitk_vec_fits(const GemmProblem& p) {
  if (p.sak != 1 || p.sbn != 1) return false;
  if ((p.K % 4) != 0 || (p.N % 4) != 0) return false;
  if ((p.sam % 4) != 0 || (p.sbk % 4) != 0 || (p.sab % 4) != 0 || (p.sbb % 4) != 0) return false;
  if ((reinterpret_cast<uintptr_t>(p.A) & 15u) != 0 || (reinterpret_cast<uintptr_t>(p.B) & 15u) != 0) return false;
  return true;
}

}  // namespace

bool f32_mfma_supported(const GemmProblem& p) {
  if (p.dtype != srtReal32F) return false;
  if (p.K < 1) return false;
  if ((p.M + 31) / 32 > 65535 || p.batch > 65535) return false;
  return true;
}

// The split-K variant pays when 64 x 64 tiles alone would leave most CUs idle.
bool f32_mfma_prefers_splitk(const GemmProblem& p) {
  const long long tiles64 = (long long)((p.M + FT - 1) / FT) * ((p.N + FT - 1) / FT) * p.batch;
  return tiles64 < 192 && p.K >= 64;
}

hipError_t launch_f32_mfma_variant(const GemmProblem& p, bool splitk, hipStream_t stream) {
  if (splitk) {
    dim3 grid((p.N + 31) / 32, (p.M + 31) / 32, p.batch);
    if (splitk_vec_fits(p)) hipLaunchKernelGGL(gemm_f32_mfma_splitk_vec_kernel, grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL(gemm_f32_mfma_splitk_kernel, grid, dim3(256), 0, stream, p);
  } else {
    if ((p.M + FT - 1) / FT > 65535) return hipErrorInvalidValue;
    dim3 grid((p.N + FT - 1) / FT, (p.M + FT - 1) / FT, p.batch);
    hipLaunchKernelGGL(gemm_f32_mfma_kernel, grid, dim3(256), 0, stream, p);
  }
  return hipGetLastError();
}

hipError_t launch_f32_mfma(const GemmProblem& p, hipStream_t stream) {
  return launch_f32_mfma_variant(p, f32_mfma_prefers_splitk(p), stream);
}

}  // namespace srt
