// fp32 matmul on the matrix cores: v_mfma_f32_32x32x2_f32 (true fp32 products and sums, no
// reduced-precision path), any strides.  Operands are staged through LDS k-major ([k][m],
// [k][n]) so the MFMA operand of lane l (row / column l % 32, k = 2 kk + l / 32) is a
// conflict-free LDS read; the next k tile is prefetched into registers while the current one
// multiplies.  Four kernels:
//
//   128 x 128, vector   every operand has a unit stride along k or m / n with 16-byte aligned rows:
//                       16-byte global loads, 8-byte operand reads (4096^3: ~120 TFLOP/s)
//   128 x 128 / 64 x 64 element-wise loads with the caller's strides (views, column-major, odd
//                       pitches all land here); the small tile when the large one would leave CUs idle
//   32 x 32 split-K     launch-latency-sized problems (512^3 = 64 tiles of 64 x 64): the 4 waves split
//                       K between them and sum through LDS; row-major operands take a variant that
//                       keeps a wave's whole k range in flight
#include "gemm_common.h"
#include "gemm_f32_ring.h"

namespace srt {

namespace {

typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4v_t __attribute__((ext_vector_type(4)));

constexpr int FT = 64;   // tile edge
constexpr int FK = 16;   // k per stage

// ---- 64 x 64 or 128 x 128 tiles, waves 2 x 2 -----------------------------------------------------
// TW = 32 x 32 MFMA tiles per wave and dimension: 1 -> 64 x 64 per workgroup, 2 -> 128 x 128.
// The fixed cost of a k stage (global loads, LDS writes, two barriers) is the same for both,
// so the large tile, with four times the MFMAs per stage, is the one that approaches the matrix
// more efficient one (4096^3: 87 -> 96 TFLOP/s); the small one is for problems that would
// otherwise leave CUs idle.
template <int TW>
__global__ __launch_bounds__(256) void gemm_f32_mfma_kernel(GemmProblem p) {
  constexpr int TILE = FT * TW;          // 64 or 128
  constexpr int PER = 4 * TW;            // elements of each operand a thread stages per k tile
  __shared__ float As[2][FK][TILE + 4];
  __shared__ float Bs[2][FK][TILE + 4];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave >> 1) * 32 * TW, wn = (wave & 1) * 32 * TW;
  const int r = lane & 31, kh = lane >> 5;
  const int m0 = blockIdx.y * TILE, n0 = blockIdx.x * TILE, bz = blockIdx.z;
  const float* A = (const float*)p.A + (long long)bz * p.sab;
  const float* B = (const float*)p.B + (long long)bz * p.sbb;
  float* C = (float*)p.C + (long long)bz * p.scb;

  // thread -> element mapping that walks the unit stride first
  const bool a_k_fast = (p.sak == 1), b_n_fast = (p.sbn == 1);
  int am[PER], ak[PER], bn[PER], bk[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int idx = tid + i * 256;
    if (a_k_fast) { ak[i] = idx & (FK - 1); am[i] = idx >> 4; } else { am[i] = idx & (TILE - 1); ak[i] = idx / TILE; }
    if (b_n_fast) { bn[i] = idx & (TILE - 1); bk[i] = idx / TILE; } else { bk[i] = idx & (FK - 1); bn[i] = idx >> 4; }
  }
  auto fetch = [&](int k0, float (&ra)[PER], float (&rb)[PER]) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int m = m0 + am[i], ka = k0 + ak[i], n = n0 + bn[i], kb = k0 + bk[i];
      ra[i] = (m < p.M && ka < p.K) ? A[(long long)m * p.sam + (long long)ka * p.sak] : 0.0f;
      rb[i] = (n < p.N && kb < p.K) ? B[(long long)kb * p.sbk + (long long)n * p.sbn] : 0.0f;
    }
  };
  auto stash = [&](int buf, const float (&ra)[PER], const float (&rb)[PER]) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      As[buf][ak[i]][am[i]] = ra[i];
      Bs[buf][bk[i]][bn[i]] = rb[i];
    }
  };

  f32x16_t acc[TW][TW];
#pragma unroll
  for (int i = 0; i < TW; ++i)
#pragma unroll
    for (int j = 0; j < TW; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  float ra[PER], rb[PER];
  fetch(0, ra, rb);
  stash(0, ra, rb);
  __syncthreads();
  const int KT = (p.K + FK - 1) / FK;
  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT) fetch((kt + 1) * FK, ra, rb);
#pragma unroll
    for (int kk = 0; kk < FK / 2; ++kk) {
      float af[TW], bf[TW];
#pragma unroll
      for (int i = 0; i < TW; ++i) af[i] = As[buf][2 * kk + kh][wm + 32 * i + r];
#pragma unroll
      for (int j = 0; j < TW; ++j) bf[j] = Bs[buf][2 * kk + kh][wn + 32 * j + r];
#pragma unroll
      for (int i = 0; i < TW; ++i)
#pragma unroll
        for (int j = 0; j < TW; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < KT) stash(buf ^ 1, ra, rb);
    __syncthreads();
  }

  // lane holds column r and rows 8 (v / 4) + 4 kh + v % 4 of each 32 x 32 tile
  Epilogue<F32> ep(p);
#pragma unroll
  for (int j = 0; j < TW; ++j) {
    const int n = n0 + wn + 32 * j + r;
    if (n >= p.N) continue;
#pragma unroll
    for (int i = 0; i < TW; ++i) {
      const int mb = m0 + wm + 32 * i + 4 * kh;
      float out[16];
#pragma unroll
      for (int v = 0; v < 16; ++v) out[v] = acc[i][j][v];
      ep.finish_run(out, [&](int v, int* m, int* nn) {
        *m = mb + 8 * (v >> 2) + (v & 3);
        *nn = n;
        return *m < p.M;
      });
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = mb + 8 * (v >> 2) + (v & 3);
        if (m < p.M) C[(long long)m * p.scm + (long long)n * p.scn] = out[v];
      }
    }
  }
}

// ---- 128 x 128 tiles, unit-stride operands: 16-byte loads, 8-byte LDS operand reads ------------
// The kernel above spends about as many issue cycles on scalar loads, address arithmetic and
// 4-byte LDS traffic as on MFMAs.  When every operand has a unit stride along k (K_FAST) or along
// m / n, 16-byte aligned rows and an extent along that stride that is a multiple of 4, a thread
// stages two 16-byte vectors per operand and k tile, and the wave's 64 x 64 tile is laid out so
// that the operands of both of its MFMA tiles along a dimension are neighbours in LDS:
//   LDS     k-major [16 k][128 mn], pitch 132.  A vector along mn is one ds_write_b128; a vector
//           along k is four ds_write_b32 (conflict-free: the lanes of a wave cover 16 rows x 4 k
//           groups, and 16 kq + row spans the 64 banks).
//   MFMA    tile (i, j) of a wave takes rows wm + 2 r + i and columns wn + 2 r + j (lane r):
//           one ds_read_b64 per operand and k pair feeds both tiles, and the two results a lane
//           holds for a row are neighbouring columns of C (one 8-byte store).
// 4096^3: 117-121 TFLOP/s for the four transpose combinations (96 with the kernel above).
template <bool K_FAST>
struct VecStage {
  f32x4v_t v[2];
  const float* ptr[2];
  int mn[2], k[2];
  bool ok[2];

  // mn0: first row / column of the tile; extent: M or N; ld: stride of the other dimension
  __device__ __forceinline__ void init(const float* base, int tid, int mn0, int extent, long long ld) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int f = tid + 256 * i;
      if (K_FAST) { mn[i] = f >> 2; k[i] = (f & 3) * 4; } else { k[i] = f >> 5; mn[i] = (f & 31) * 4; }
      ok[i] = mn0 + mn[i] < extent;   // the extent along a unit stride is a multiple of 4: whole vectors
      ptr[i] = K_FAST ? base + (long long)(mn0 + mn[i]) * ld + k[i] : base + (long long)k[i] * ld + mn0 + mn[i];
    }
  }
  __device__ __forceinline__ void load(int k0, int K, long long ld) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const f32x4v_t zero = {0.0f, 0.0f, 0.0f, 0.0f};
      const float* q = K_FAST ? ptr[i] + k0 : ptr[i] + (long long)k0 * ld;
      v[i] = (ok[i] && k0 + k[i] < K) ? *reinterpret_cast<const f32x4v_t*>(q) : zero;
    }
  }
  __device__ __forceinline__ void store(float (*dst)[132]) const {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if (K_FAST) {
#pragma unroll
        for (int e = 0; e < 4; ++e) dst[k[i] + e][mn[i]] = v[i][e];
      } else {
        *reinterpret_cast<f32x4v_t*>(&dst[k[i]][mn[i]]) = v[i];
      }
    }
  }
};

typedef float f32x2v_t __attribute__((ext_vector_type(2)));

template <bool A_KF, bool B_KF>
__global__ __launch_bounds__(256) void gemm_f32_mfma128_vec_kernel(GemmProblem p) {
  __shared__ __attribute__((aligned(16))) float As[2][FK][132];
  __shared__ __attribute__((aligned(16))) float Bs[2][FK][132];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
  const int r = lane & 31, kh = lane >> 5;
  const int m0 = blockIdx.y * 128, n0 = blockIdx.x * 128, bz = blockIdx.z;
  const float* A = (const float*)p.A + (long long)bz * p.sab;
  const float* B = (const float*)p.B + (long long)bz * p.sbb;
  float* C = (float*)p.C + (long long)bz * p.scb;
  const long long lda = A_KF ? p.sam : p.sak, ldb = B_KF ? p.sbn : p.sbk;

  VecStage<A_KF> sa;
  VecStage<B_KF> sb;
  sa.init(A, tid, m0, p.M, lda);
  sb.init(B, tid, n0, p.N, ldb);

  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  sa.load(0, p.K, lda);
  sb.load(0, p.K, ldb);
  sa.store(As[0]);
  sb.store(Bs[0]);
  __syncthreads();
  const int KT = (p.K + FK - 1) / FK;
  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT) {
      sa.load((kt + 1) * FK, p.K, lda);
      sb.load((kt + 1) * FK, p.K, ldb);
    }
#pragma unroll
    for (int kk = 0; kk < FK / 2; ++kk) {
      const f32x2v_t af = *reinterpret_cast<const f32x2v_t*>(&As[buf][2 * kk + kh][wm + 2 * r]);
      const f32x2v_t bf = *reinterpret_cast<const f32x2v_t*>(&Bs[buf][2 * kk + kh][wn + 2 * r]);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < KT) {
      sa.store(As[buf ^ 1]);
      sb.store(Bs[buf ^ 1]);
    }
    __syncthreads();
  }

  // tile (i, j): lane r holds column wn + 2 r + j and rows wm + 2 (8 (v / 4) + 4 kh + v % 4) + i
  Epilogue<F32> ep(p);
  const int n = n0 + wn + 2 * r;
  const bool pair_store = p.scn == 1 && (p.scm % 2) == 0 && (p.scb % 2) == 0 &&
                          (reinterpret_cast<uintptr_t>(p.C) & 7u) == 0 && n + 1 < p.N;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    float out[2][16];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int v = 0; v < 16; ++v) out[j][v] = acc[i][j][v];
      ep.finish_run(out[j], [&](int v, int* m, int* nn) {
        *m = m0 + wm + 2 * (8 * (v >> 2) + 4 * kh + (v & 3)) + i;
        *nn = n + j;
        return *m < p.M && *nn < p.N;
      });
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int m = m0 + wm + 2 * (8 * (v >> 2) + 4 * kh + (v & 3)) + i;
      if (m >= p.M) continue;
      const float c0 = out[0][v], c1 = out[1][v];
      if (pair_store) {
        const f32x2v_t c = {c0, c1};
        *reinterpret_cast<f32x2v_t*>(C + (long long)m * p.scm + n) = c;
      } else {
        if (n < p.N) C[(long long)m * p.scm + (long long)n * p.scn] = c0;
        if (n + 1 < p.N) C[(long long)m * p.scm + (long long)(n + 1) * p.scn] = c1;
      }
    }
  }
}

// Preconditions of the 128 x 128 vector kernel: unit stride along k or along m / n for both
// operands, 16-byte aligned rows, whole 16-byte vectors along the unit stride.
bool mfma128_vec_fits(const GemmProblem& p) {
  const bool a_kf = p.sak == 1, a_mf = p.sam == 1;
  const bool b_kf = p.sbk == 1, b_nf = p.sbn == 1;
  if (!(a_kf || a_mf) || !(b_kf || b_nf)) return false;
  const long long lda = a_kf ? p.sam : p.sak, ldb = b_kf ? p.sbn : p.sbk;
  if ((lda % 4) != 0 || (ldb % 4) != 0 || (p.sab % 4) != 0 || (p.sbb % 4) != 0) return false;
  if ((a_kf ? p.K : p.M) % 4 != 0 || (b_kf ? p.K : p.N) % 4 != 0) return false;
  if ((reinterpret_cast<uintptr_t>(p.A) & 15u) != 0 || (reinterpret_cast<uintptr_t>(p.B) & 15u) != 0) return false;
  return true;
}

hipError_t launch_mfma128_vec(const GemmProblem& p, hipStream_t stream) {
  dim3 grid((p.N + 127) / 128, (p.M + 127) / 128, p.batch);
  const bool a_kf = p.sak == 1, b_kf = p.sbk == 1 && p.sbn != 1;
  // an operand with both strides 1 (a single row or column) counts as k-contiguous for A, n-contiguous for B
  if (a_kf && b_kf) hipLaunchKernelGGL((gemm_f32_mfma128_vec_kernel<true, true>), grid, dim3(256), 0, stream, p);
  else if (a_kf) hipLaunchKernelGGL((gemm_f32_mfma128_vec_kernel<true, false>), grid, dim3(256), 0, stream, p);
  else if (b_kf) hipLaunchKernelGGL((gemm_f32_mfma128_vec_kernel<false, true>), grid, dim3(256), 0, stream, p);
  else hipLaunchKernelGGL((gemm_f32_mfma128_vec_kernel<false, false>), grid, dim3(256), 0, stream, p);
  return launch_status(stream);
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
  const int mb = m0 + 8 * wave + 4 * kh;
  float out[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int v = 4 * wave + i;
    out[i] = (red[0][v][lane] + red[1][v][lane]) + (red[2][v][lane] + red[3][v][lane]);
  }
  ep.finish_run(out, [&](int i, int* m, int* nn) {
    *m = mb + i;
    *nn = n;
    return *m < p.M;
  });
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (mb + i < p.M) C[(long long)(mb + i) * p.scm + (long long)n * p.scn] = out[i];
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
  const int mb = m0 + 8 * wave + 4 * kh;
  float out[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int v = 4 * wave + i;
    out[i] = (red[0][v][lane] + red[1][v][lane]) + (red[2][v][lane] + red[3][v][lane]);
  }
  ep.finish_run(out, [&](int i, int* m, int* nn) {
    *m = mb + i;
    *nn = n;
    return *m < p.M;
  });
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (mb + i < p.M) C[(long long)(mb + i) * p.scm + (long long)n * p.scn] = out[i];
}

// Preconditions of the vector variant: both operands row-major with 16-byte aligned rows.
bool splitk_vec_fits(const GemmProblem& p) {
  if (p.sak != 1 || p.sbn != 1) return false;
  if ((p.K % 4) != 0 || (p.N % 4) != 0) return false;
  if ((p.sam % 4) != 0 || (p.sbk % 4) != 0 || (p.sab % 4) != 0 || (p.sbb % 4) != 0) return false;
  if ((reinterpret_cast<uintptr_t>(p.A) & 15u) != 0 || (reinterpret_cast<uintptr_t>(p.B) & 15u) != 0) return false;
  return true;
}

// ---- split-K over the 128 x 128 vector kernel -----------------------------------------------------
// The 128 x 128 kernel leans on several workgroups per compute unit to hide its k stages' load latency and barriers
// (4096^3, four per unit: 117-121 TFLOP/s; 2048^3, one per unit: 92), and a problem of fewer tiles than units
// leaves units idle on top (512 x 4096 x 4096: 128 tiles).  Such a problem's k range is cut into S equal parts that
// run as S "batches" of the kernel (operand batch stride = one part's k extent), each storing its accumulators to a
// workspace [S][M][N]; a second kernel adds the parts in a fixed order and applies bias and activation.  fp32
// throughout; the result does not depend on timing.
__global__ __launch_bounds__(256) void f32_parts_reduce_kernel(const float* part, int parts, GemmProblem p) {
  const int n4 = (p.N + 3) / 4;   // one lane per four consecutive columns
  const long long id = (long long)blockIdx.x * 256 + threadIdx.x;
  if (id >= (long long)p.M * n4) return;
  const int m = (int)(id / n4), n = (int)(id - (long long)m * n4) * 4;
  const long long mn = (long long)p.M * p.N;
  const float* src = part + (long long)m * p.N + n;
  float* C = (float*)p.C;
  Epilogue<F32> ep(p);
  if ((p.N & 3) == 0) {   // the workspace's rows are 16-byte aligned
    f32x4v_t sum = *reinterpret_cast<const f32x4v_t*>(src);
    for (int s = 1; s < parts; ++s) sum += *reinterpret_cast<const f32x4v_t*>(src + s * mn);
    float out[4] = {sum[0], sum[1], sum[2], sum[3]};
    ep.finish_run(out, [&](int e, int* mm, int* nn) {
      *mm = m;
      *nn = n + e;
      return true;
    });
    if (p.scn == 1 && (p.scm & 3) == 0 && (reinterpret_cast<uintptr_t>(C) & 15u) == 0) {
      const f32x4v_t o = {out[0], out[1], out[2], out[3]};
      *reinterpret_cast<f32x4v_t*>(C + (long long)m * p.scm + n) = o;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) C[(long long)m * p.scm + (long long)(n + e) * p.scn] = out[e];
    }
  } else {
    for (int e = 0; e < 4 && n + e < p.N; ++e) {
      float sum = src[e];
      for (int s = 1; s < parts; ++s) sum += src[e + s * mn];
      C[(long long)m * p.scm + (long long)(n + e) * p.scn] = ep.finish(sum, ep.bias_at(m, n + e));
    }
  }
}

}  // namespace

// ---- the 128 x 128 ring kernel (gemm_f32_ring.h) ----------------------------------------------------
// Preconditions: both operands contiguous along k or along m / n with 16-byte aligned rows and whole 16-byte vectors,
// K in whole 64-deep units (at least two), 32-bit byte offsets that reach every operand (rows of a partial last tile
// included).
bool f32_ring_fits(const GemmProblem& p) {
  if (p.dtype != srtReal32F || !mfma128_vec_fits(p)) return false;
  if (p.K % f32r::DK != 0 || p.K < 2 * f32r::DK) return false;
  if (p.batch > 65535 || p.sab < 0 || p.sbb < 0 || p.sam < 0 || p.sak < 0 || p.sbk < 0 || p.sbn < 0 || p.scm < 0 || p.scn < 0) return false;
  const bool a_kc = p.sak == 1, b_kc = p.sbk == 1 && p.sbn != 1;
  const long long lda = a_kc ? p.sam : p.sak, ldb = b_kc ? p.sbn : p.sbk;
  const long long nb = p.batch - 1;
  const long long a_reach = nb * p.sab + (a_kc ? ((long long)p.M + 128) * lda + p.K : ((long long)p.K + 64) * lda + p.M + 128);
  const long long b_reach = nb * p.sbb + (b_kc ? ((long long)p.N + 128) * ldb + p.K : ((long long)p.K + 64) * ldb + p.N + 128);
  const long long lim = 0x7fffffffLL / 4 - 4096;   // in elements: byte offsets stay below 2^31
  if (!(a_reach < lim && b_reach < lim)) return false;
  const long long tiles = (long long)((p.M + 127) / 128) * ((p.N + 127) / 128) * p.batch;
  return tiles < (1LL << 30);
}

// shape 0: 128 x 128 tiles, 1: 64 x 128, 2: 64 x 64 (the same kernel with one MFMA tile per wave along m, or along both)
hipError_t launch_f32_ring(const GemmProblem& p, hipStream_t stream, int shape) {
  const bool a_kc = p.sak == 1, b_kc = p.sbk == 1 && p.sbn != 1;
  constexpr int lds_bytes = f32r::UNITS * f32r::UNIT;
  const int tile_m = shape == 0 ? 128 : 64, tile_n = shape == 2 ? 64 : 128;
  const long long tiles = (long long)((p.M + tile_m - 1) / tile_m) * ((p.N + tile_n - 1) / tile_n) * p.batch;
  const int grid = ring::persistent_grid(tiles);
  auto go = [&](auto kernel, std::atomic<uint32_t>& configured) {
    if (hipError_t e = ensure_lds_limit(reinterpret_cast<const void*>(kernel), lds_bytes, configured); e != hipSuccess) return e;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(ring::NT), lds_bytes, stream, p);
    return launch_status(stream);
  };
  static std::atomic<uint32_t> configured[3][4];
  auto layout = [&](auto tm, auto tn, std::atomic<uint32_t>* c) {
    constexpr int TM = decltype(tm)::value, TN = decltype(tn)::value;
    if (a_kc && b_kc) return go(f32r::gemm_f32_ring_kernel<true, true, TM, TN>, c[3]);
    if (a_kc) return go(f32r::gemm_f32_ring_kernel<true, false, TM, TN>, c[2]);
    if (b_kc) return go(f32r::gemm_f32_ring_kernel<false, true, TM, TN>, c[1]);
    return go(f32r::gemm_f32_ring_kernel<false, false, TM, TN>, c[0]);
  };
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  if (shape == 0) return layout(I2{}, I2{}, configured[0]);
  if (shape == 1) return layout(I1{}, I2{}, configured[1]);
  if (shape == 2) return layout(I1{}, I1{}, configured[2]);
  return hipErrorInvalidValue;
}

// Parts the k range of `p` is cut into for the pass above, or 0 when the problem does not take it: a single matrix
// of more than 64 rows (fewer: the 32 x 32 kernel) whose operands the 128 x 128 kernels read, and too few tiles.
// On the ring kernel (parts of whole 64-deep units, at least two each) the count comes from an estimate of the time,
// in microseconds: rounds of the persistent grid x 59 per 1024 k of a part (a 128 x 128 tile at nine tenths of a
// unit's fp32 matrix rate) + 4, and for S > 1 parts the sums, S x M x N x 8 bytes at 6 TB/s, + 5 for the second
// launch.  Measured / estimated: 512 x 4096 x 4096 whole 236 / 240, in two 129 / 133; 256 x 8192 x 8192 in two 258 / 251.
// More parts must buy a tenth to be taken.  The register-staged kernel wants two workgroups per unit and parts of at
// least 256.
int f32_tile_parts(const GemmProblem& p) {
  if (p.dtype != srtReal32F || p.batch != 1 || p.M <= 64 || p.K < 256) return 0;
  if (!mfma128_vec_fits(p) || (p.M + 127) / 128 > 65535) return 0;
  if ((long long)p.M * p.N >= (1LL << 31)) return 0;
  const long long tiles = (long long)((p.M + 127) / 128) * ((p.N + 127) / 128);
  const int cus = compute_units();
  if (f32_ring_fits(p)) {
    if (tiles >= cus) return 0;
    int best = 1;
    double best_us = 0.0;
    for (int s = 1; s <= 16; s *= 2) {
      if (p.K % (s * f32r::DK) != 0 || p.K / s < 2 * f32r::DK) break;
      const double rounds = (double)((tiles * s + cus - 1) / cus);
      double us = rounds * 59.0 * (double)(p.K / s) / 1024.0 + 4.0;
      if (s > 1) us += (double)s * (double)p.M * (double)p.N * 8.0 / 6.0e6 + 5.0;
      if (s == 1 || us < 0.9 * best_us) {
        best = s;
        best_us = us;
      }
    }
    return best >= 2 ? best : 0;
  }
  const long long want = 2LL * cus;
  if (tiles >= want) return 0;
  int parts = 0;
  for (int s = 2; s <= 16; s *= 2) {
    if (p.K % (s * FK) != 0 || p.K / s < 256) break;
    parts = s;
    if (tiles * s >= want) break;
  }
  return parts;
}

hipError_t launch_f32_tile_parts(const GemmProblem& p, hipStream_t stream) {
  const int parts = f32_tile_parts(p);
  if (parts < 2) return hipErrorInvalidValue;
  void* workspace = nullptr;
  const size_t bytes = (size_t)parts * p.M * p.N * sizeof(float);
  if (srtDeviceAllocate(&workspace, bytes, reinterpret_cast<srtStream>(stream)) != srtSuccess) return hipErrorOutOfMemory;
  GemmProblem q = p;
  q.K = p.K / parts;
  q.batch = parts;
  q.sab = (long long)q.K * p.sak;   // part s starts q.K further along k
  q.sbb = (long long)q.K * p.sbk;
  q.C = workspace;
  q.scm = p.N;
  q.scn = 1;
  q.scb = (long long)p.M * p.N;
  q.bias = nullptr;
  q.activation = srtActivationIdentity;
  hipError_t e = f32_ring_fits(q) ? launch_f32_ring(q, stream, 0) : launch_mfma128_vec(q, stream);
  if (e == hipSuccess) {
    const long long lanes = (long long)p.M * ((p.N + 3) / 4);
    hipLaunchKernelGGL(f32_parts_reduce_kernel, dim3((unsigned)((lanes + 255) / 256)), dim3(256), 0, stream,
                       (const float*)workspace, parts, p);
    e = launch_status(stream);
  }
  (void)srtDeviceFree(workspace);   // stream-ordered: reused only by work queued after the kernels above
  return e;
}

bool f32_mfma_supported(const GemmProblem& p) {
  if (p.dtype != srtReal32F) return false;
  if (p.K < 1) return false;
  if ((p.M + 31) / 32 > 65535 || p.batch > 65535) return false;
  return true;
}

// Which fp32 kernel a problem the ring kernel reads should run on, by estimates of the time in microseconds (each
// fitted to measurements on one device, 256 units; R(t) = rounds of t tiles over the units):
//   128 x 128 tiles   R x 59 per 1024 k + 4        (2048^3 124 / 122, 1024 x 4096 x 4096 239 / 240, 1536^3 92 / 92)
//   64 x 128 tiles    R x 30.5 per 1024 k + 4      (512 x 4096 x 4096 125 / 126, 256 x 8192 x 8192 255 / 248, 1536^3 95 / 96)
//   64 x 64 tiles     R x 16.5 per 1024 k + 4      (1024^3 20.3 / 20.5, 64 x 14336 x 4096 71 / 70, 1536^3 77 / 78, 768^3 15.9 / 16.4)
//   k in parts on 128 x 128 tiles: f32_tile_parts' estimate
//   32 x 32 tiles, k split over the waves: every workgroup reads 64 x K x 4 bytes, at 32 bytes/ns alone on its unit and 31
//   per unit when they share (both operands row-major: 16-byte loads), 16 and 21.5 otherwise, + 3
//                      (512^3 6.7 / 7.1, 1024^3 31 / 37 and 42 / 52, 32 x 14336 x 4096 59 / 62 and 90 / 88, 128 x 512 x 4096 35 / 36 and 68 / 69)
// Smaller tiles cost more per flop (more operand bytes per MFMA through L2 and LDS) and win by filling the device:
// 1024^3 20 us on 256 tiles of 64 x 64 against 31-42 on 32 x 32 and 62 on 64 tiles of 128 x 128.
// Returns 0: 128 x 128, 1: 64 x 128, 2: 64 x 64, 3: parts, 4: the 32 x 32 kernel.
int f32_ring_choice(const GemmProblem& p) {
  const int cus = compute_units();
  auto rounds = [&](int tm, int tn) {
    const long long t = (long long)((p.M + tm - 1) / tm) * ((p.N + tn - 1) / tn) * p.batch;
    return (double)((t + cus - 1) / cus);
  };
  const double k = (double)p.K / 1024.0;
  double best = rounds(128, 128) * 59.0 * k + 4.0;
  int choice = 0;
  auto offer = [&](int c, double us) {
    if (us < best) {
      best = us;
      choice = c;
    }
  };
  offer(1, rounds(64, 128) * 30.5 * k + 4.0);
  offer(2, rounds(64, 64) * 16.5 * k + 4.0);
  if (const int s = f32_tile_parts(p); s >= 2) {
    const long long tiles = (long long)((p.M + 127) / 128) * ((p.N + 127) / 128);
    offer(3, (double)((tiles * s + cus - 1) / cus) * 59.0 * (double)(p.K / s) / 1024.0 + 4.0 +
                 (double)s * (double)p.M * (double)p.N * 8.0 / 6.0e6 + 5.0);
  }
  if (f32_mfma_supported(p)) {
    const double tiles32 = (double)((p.M + 31) / 32) * (double)((p.N + 31) / 32) * (double)p.batch;
    const double bytes = 64.0 * (double)p.K * 4.0;   // per workgroup
    const bool vec = splitk_vec_fits(p);
    const double alone = bytes / (vec ? 32.0e3 : 16.0e3), shared = tiles32 / cus * bytes / (vec ? 31.0e3 : 21.5e3);
    offer(4, (alone > shared ? alone : shared) + 3.0);
  }
  return choice;
}


// The split-K variant pays when 64 x 64 tiles alone would leave most CUs idle.
// With up to 64 rows it pays whatever the tile count: larger tiles would be mostly padding (32 x 14336 x 4096: 60 us
// against 181 in 64 x 64 tiles).
bool f32_mfma_prefers_splitk(const GemmProblem& p) {
  const long long tiles64 = (long long)((p.M + FT - 1) / FT) * ((p.N + FT - 1) / FT) * p.batch;
  return (tiles64 <= 256 || p.M <= 64) && p.K >= 64;   // (1024^3, 256 tiles: 33 us against 43 in parts and 49 in 64 x 64 tiles)
}

hipError_t launch_f32_mfma_variant(const GemmProblem& p, bool splitk, hipStream_t stream) {
  if (splitk) {
    dim3 grid((p.N + 31) / 32, (p.M + 31) / 32, p.batch);
    if (splitk_vec_fits(p)) hipLaunchKernelGGL(gemm_f32_mfma_splitk_vec_kernel, grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL(gemm_f32_mfma_splitk_kernel, grid, dim3(256), 0, stream, p);
  } else {
    // the 128 x 128 tile once it gives every CU a workgroup, the 64 x 64 tile below that
    const long long tiles128 = (long long)((p.M + 127) / 128) * ((p.N + 127) / 128) * p.batch;
    if (tiles128 >= 256) {
      if ((p.M + 127) / 128 > 65535) return hipErrorInvalidValue;
      if (mfma128_vec_fits(p)) return launch_mfma128_vec(p, stream);
      dim3 grid((p.N + 127) / 128, (p.M + 127) / 128, p.batch);
      hipLaunchKernelGGL(gemm_f32_mfma_kernel<2>, grid, dim3(256), 0, stream, p);
    } else {
      if ((p.M + FT - 1) / FT > 65535) return hipErrorInvalidValue;
      dim3 grid((p.N + FT - 1) / FT, (p.M + FT - 1) / FT, p.batch);
      hipLaunchKernelGGL(gemm_f32_mfma_kernel<1>, grid, dim3(256), 0, stream, p);
    }
  }
  return launch_status(stream);
}

hipError_t launch_f32_mfma(const GemmProblem& p, hipStream_t stream) {
  return launch_f32_mfma_variant(p, f32_mfma_prefers_splitk(p), stream);
}

}  // namespace srt
