// bf16 / fp16 matmul on the gfx950 matrix cores: v_mfma_f32_32x32x16 tiles, fp32
// accumulation in registers, double-buffered LDS staging, fused bias + activation epilogue.
//
// Work decomposition
//   grid    one workgroup per BM x BN tile of C (x batch); workgroup ids are remapped so that
//           the workgroups resident on one XCD (ids congruent mod 8) cover a compact patch of
//           tiles and share A row panels / B column panels in that XCD's L2.
//   block   4 waves in a 2 x 2 arrangement; each wave owns (BM/2) x (BN/2) of the tile as
//           TM x TN MFMA tiles of 32 x 32, i.e. TM*TN*16 fp32 accumulators per lane.
//   k loop  BK = 64 per stage; global loads for stage t+1 are issued before the MFMAs of
//           stage t and written to the other LDS buffer afterwards (one barrier per stage).
//
// LDS layout (both operands, all four transpose cases): row r of the tile (an m for A, an n
// for B) holds its 64 k-values contiguously (128 bytes) as eight 16-byte chunks; chunk c is
// stored at position c ^ f(r), f(r) = ((r >> 1) ^ (r >> 4)) & 7.  An MFMA operand read is one
// ds_read_b128 per lane (lane l: row l % 32, chunk 2*kk + l / 32) and the XOR spreads the 16
// lanes that share an LDS pass over all 64 banks.  What differs per transpose flag is only how
// the tile gets there:
//   operand stored k-contiguous  (A not transposed / B transposed): 16-byte global loads along
//       k, written to LDS as they are;
//   operand stored mn-contiguous (A transposed / B not transposed): each thread loads an
//       8(k) x 8(mn) block as eight 16-byte rows (coalesced along mn), transposes it in
//       registers with 32 v_perm_b32 and writes eight k-contiguous chunks;
//   operand with a unit stride that misses the alignment rules (odd extents or leading strides,
//       a base that is not 16-byte aligned): the same two loaders with 16-byte loads at 2-byte
//       alignment (global memory takes them), and element loads for the one chunk per row that
//       would cross the end of the contiguous dimension;
//   operand with non-unit strides in both dimensions: 2-byte loads with arbitrary element strides,
//       eight k-values of a row packed into one chunk in registers.
#include "gemm_common.h"

namespace srt {

// 256 x 256 ring kernels, one translation unit per (type, layout): gemm_ring_inst.hip
bool ring_fits_problem(const GemmProblem& p, bool a_kc, bool b_kc);
hipError_t launch_kc64_BF16(const GemmProblem& p, hipStream_t stream);
hipError_t launch_kc64_F16(const GemmProblem& p, hipStream_t stream);
#define SRT_RING_DECL(T) \
  hipError_t launch_ring_##T##_00(const GemmProblem&, hipStream_t); \
  hipError_t launch_ring_##T##_01(const GemmProblem&, hipStream_t); \
  hipError_t launch_ring_##T##_10(const GemmProblem&, hipStream_t); \
  hipError_t launch_ring_##T##_11(const GemmProblem&, hipStream_t);
SRT_RING_DECL(BF16)
SRT_RING_DECL(F16)
#undef SRT_RING_DECL
#define SRT_M16_DECL(T)                                                  \
  hipError_t launch_m16_##T##_00(const GemmProblem&, hipStream_t);       \
  hipError_t launch_m16_##T##_01(const GemmProblem&, hipStream_t);       \
  hipError_t launch_m16_##T##_10(const GemmProblem&, hipStream_t);       \
  hipError_t launch_m16_##T##_11(const GemmProblem&, hipStream_t);
SRT_M16_DECL(BF16)
SRT_M16_DECL(F16)
#undef SRT_M16_DECL
#define SRT_M16P_DECL(T)                                                         \
  hipError_t launch_m16_partial_##T##_00(const GemmProblem&, hipStream_t);       \
  hipError_t launch_m16_partial_##T##_01(const GemmProblem&, hipStream_t);       \
  hipError_t launch_m16_partial_##T##_10(const GemmProblem&, hipStream_t);       \
  hipError_t launch_m16_partial_##T##_11(const GemmProblem&, hipStream_t);
SRT_M16P_DECL(BF16)
SRT_M16P_DECL(F16)
#undef SRT_M16P_DECL
#define SRT_M16D_DECL(T)                                                  \
  hipError_t launch_m16d_##T##_00(const GemmProblem&, hipStream_t);       \
  hipError_t launch_m16d_##T##_01(const GemmProblem&, hipStream_t);       \
  hipError_t launch_m16d_##T##_10(const GemmProblem&, hipStream_t);       \
  hipError_t launch_m16d_##T##_11(const GemmProblem&, hipStream_t);
SRT_M16D_DECL(BF16)
SRT_M16D_DECL(F16)
#undef SRT_M16D_DECL
#define SRT_M16DT_DECL(T)                                                      \
  hipError_t launch_m16d_tail_##T##_00(const GemmProblem&, hipStream_t);       \
  hipError_t launch_m16d_tail_##T##_01(const GemmProblem&, hipStream_t);       \
  hipError_t launch_m16d_tail_##T##_10(const GemmProblem&, hipStream_t);       \
  hipError_t launch_m16d_tail_##T##_11(const GemmProblem&, hipStream_t);
SRT_M16DT_DECL(BF16)
SRT_M16DT_DECL(F16)
#undef SRT_M16DT_DECL
#define SRT_M16DP_DECL(T)                                                         \
  hipError_t launch_m16d_partial_##T##_00(const GemmProblem&, hipStream_t);       \
  hipError_t launch_m16d_partial_##T##_01(const GemmProblem&, hipStream_t);       \
  hipError_t launch_m16d_partial_##T##_10(const GemmProblem&, hipStream_t);       \
  hipError_t launch_m16d_partial_##T##_11(const GemmProblem&, hipStream_t);
SRT_M16DP_DECL(BF16)
SRT_M16DP_DECL(F16)
#undef SRT_M16DP_DECL
bool m16d_tail_fits_BF16_xx(const GemmProblem&);   // (the answer does not depend on the element type)
#define SRT_M16DS_DECL(T)                                                       \
  hipError_t launch_m16d_split_##T##_00(const GemmProblem&, hipStream_t);       \
  hipError_t launch_m16d_split_##T##_01(const GemmProblem&, hipStream_t);       \
  hipError_t launch_m16d_split_##T##_10(const GemmProblem&, hipStream_t);       \
  hipError_t launch_m16d_split_##T##_11(const GemmProblem&, hipStream_t);
SRT_M16DS_DECL(BF16)
SRT_M16DS_DECL(F16)
#undef SRT_M16DS_DECL
bool m16d_split_fits_BF16_xx(const GemmProblem&);
hipError_t launch_m16dh_BF16_10(const GemmProblem&, hipStream_t);
hipError_t launch_m16dh_BF16_11(const GemmProblem&, hipStream_t);
hipError_t launch_m16dh_F16_10(const GemmProblem&, hipStream_t);
hipError_t launch_m16dh_F16_11(const GemmProblem&, hipStream_t);
hipError_t launch_m16dn_BF16_00(const GemmProblem&, hipStream_t);
hipError_t launch_m16dn_BF16_01(const GemmProblem&, hipStream_t);
hipError_t launch_m16dn_F16_00(const GemmProblem&, hipStream_t);
hipError_t launch_m16dn_F16_01(const GemmProblem&, hipStream_t);
hipError_t launch_m16q_BF16_00(const GemmProblem&, hipStream_t);
hipError_t launch_m16q_BF16_01(const GemmProblem&, hipStream_t);
hipError_t launch_m16q_BF16_10(const GemmProblem&, hipStream_t);
hipError_t launch_m16q_BF16_11(const GemmProblem&, hipStream_t);
hipError_t launch_m16q_F16_00(const GemmProblem&, hipStream_t);
hipError_t launch_m16q_F16_01(const GemmProblem&, hipStream_t);
hipError_t launch_m16q_F16_10(const GemmProblem&, hipStream_t);
hipError_t launch_m16q_F16_11(const GemmProblem&, hipStream_t);
hipError_t launch_m16dh_partial_BF16_11(const GemmProblem&, hipStream_t);
hipError_t launch_m16dh_partial_F16_11(const GemmProblem&, hipStream_t);
hipError_t launch_m16h_BF16_10(const GemmProblem&, hipStream_t);
hipError_t launch_m16h_BF16_11(const GemmProblem&, hipStream_t);
hipError_t launch_m16h_F16_10(const GemmProblem&, hipStream_t);
hipError_t launch_m16h_F16_11(const GemmProblem&, hipStream_t);
hipError_t launch_m16h_partial_BF16_10(const GemmProblem&, hipStream_t);
hipError_t launch_m16h_partial_BF16_11(const GemmProblem&, hipStream_t);
hipError_t launch_m16h_partial_F16_10(const GemmProblem&, hipStream_t);
hipError_t launch_m16h_partial_F16_11(const GemmProblem&, hipStream_t);

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int BK = 64;          // k depth of one LDS stage
constexpr int ROW_BYTES = 128;  // BK * 2 bytes
constexpr int NT = 256;         // threads per workgroup (4 waves)

template <typename T>
__device__ __forceinline__ f32x16_t mfma32(u32x4_t a, u32x4_t b, f32x16_t c);

template <>
__device__ __forceinline__ f32x16_t mfma32<BF16>(u32x4_t a, u32x4_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b),
                                                 c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x16_t mfma32<F16>(u32x4_t a, u32x4_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b),
                                                c, 0, 0, 0);
}

__device__ __forceinline__ int swz(int row) { return ((row >> 1) ^ (row >> 4)) & 7; }

__device__ __forceinline__ uint32_t lds_off(int row, int chunk) {
  return (uint32_t)(row * ROW_BYTES + ((chunk ^ swz(row)) << 4));
}

// ---- global -> register staging --------------------------------------------------------------
// Up to 7 elements src[0], src[stride], ... (count of them, 1..7) as the leading halves of a
// 16-byte chunk, zero behind them: the end of a contiguous dimension that is not a multiple of 8.
__device__ __forceinline__ u32x4_t load_chunk_tail(const uint16_t* src, int count) {
  uint32_t h[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) h[j] = (uint32_t)src[min(j, count - 1)] & (uint32_t)((j - count) >> 31);
  return u32x4_t{h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)};
}

// 16 bytes from an address with 2-byte alignment: still one global_load_dwordx4 (global memory
// takes it at any alignment).  Rows that are off by 2 bytes load at well under half the aligned
// rate (4096 x 4097 x 4096 with such rows of B: 186 TFLOP/s; with rows that merely miss the 16-byte
// rule: 450-560); fetching aligned dwords plus a fifth and funnel-shifting them into place was
// tried and is slower still (155 and 360-430).
__device__ __forceinline__ u32x4_t load_chunk_unaligned(const uint16_t* src) {
  u32x4_t x;
  __builtin_memcpy(&x, src, 16);
  return x;
}

// K-contiguous operand: R rows x 64 k.  Thread t owns chunk t % 8 of rows t / 8 + 32 i.
// ALIGNED: rows start on 16-byte boundaries and K is a multiple of 8.
template <int R, bool ALIGNED = true>
struct StageK {
  static constexpr int CH = R * 8 / NT;
  u32x4_t v[CH];

  __device__ __forceinline__ void load(const uint16_t* base, long long ld, long long, int row0, int rows_total, int k0,
                                       int K, int tid) {
    const int chunk = tid & 7;
    const int k = k0 + chunk * 8;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int row = row0 + (tid >> 3) + 32 * i;
      u32x4_t x = {0u, 0u, 0u, 0u};
      if (row < rows_total && k < K) {
        const uint16_t* src = base + (long long)row * ld + k;
        if (ALIGNED) {
          x = *reinterpret_cast<const u32x4_t*>(src);
        } else if (k + 8 <= K) {
          x = load_chunk_unaligned(src);
        } else {
          x = load_chunk_tail(src, K - k);
        }
      }
      v[i] = x;
    }
  }

  __device__ __forceinline__ void store(unsigned char* lds, int tid) const {
    const int chunk = tid & 7;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int row = (tid >> 3) + 32 * i;
      *reinterpret_cast<u32x4_t*>(lds + lds_off(row, chunk)) = v[i];
    }
  }
};

// MN-contiguous operand: 64 k x R mn, element (k, mn) at base[k * ld + mn].  Thread t (< R)
// owns the 8 x 8 block k-group t / (R/8), mn-group t % (R/8).
template <int R, bool ALIGNED = true>
struct StageMN {
  static constexpr int GROUPS = R / 8;
  u32x4_t v[8];

  __device__ __forceinline__ void load(const uint16_t* base, long long, long long ld, int mn0, int mn_total, int k0,
                                       int K, int tid) {
    if (R < NT && tid >= R) return;
    const int mn = mn0 + (tid % GROUPS) * 8;
    const int kb = k0 + (tid / GROUPS) * 8;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      u32x4_t x = {0u, 0u, 0u, 0u};
      if (mn < mn_total && kb + j < K) {
        const uint16_t* src = base + (long long)(kb + j) * ld + mn;
        if (ALIGNED) {
          x = *reinterpret_cast<const u32x4_t*>(src);
        } else if (mn + 8 <= mn_total) {
          x = load_chunk_unaligned(src);
        } else {
          x = load_chunk_tail(src, mn_total - mn);
        }
      }
      v[j] = x;
    }
  }

  __device__ __forceinline__ void store(unsigned char* lds, int tid) const {
    if (R < NT && tid >= R) return;
    const int g = tid % GROUPS;
    const int kg = tid / GROUPS;
    // neighbouring lanes start on rows of opposite parity so one LDS pass covers all banks:
    // at step jj a lane writes row jj ^ (g & 1).  The source dword (jj >> 1) is the same for
    // both rows of a pair; only the half-word selector depends on the lane.
    const uint32_t sel_lo = 0x05040100u, sel_hi = 0x07060302u;
    const uint32_t sel_even = (g & 1) ? sel_hi : sel_lo;  // selector used at even jj
    const uint32_t sel_odd = (g & 1) ? sel_lo : sel_hi;
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) {
      const int n = jj ^ (g & 1);
      const uint32_t sel = (jj & 1) ? sel_odd : sel_even;
      u32x4_t o;
      // o[d] = { v[2d][n] , v[2d+1][n] } as two 16-bit halves: one byte-permute per dword
#pragma unroll
      for (int d = 0; d < 4; ++d) o[d] = __builtin_amdgcn_perm(v[2 * d + 1][jj >> 1], v[2 * d][jj >> 1], sel);
      const int row = g * 8 + n;
      *reinterpret_cast<u32x4_t*>(lds + lds_off(row, kg)) = o;
    }
  }
};

// Any strides: element (mn, k) at base[mn * s_mn + k * s_k], 2-byte loads.  A thread fills whole
// chunks (8 k of one row): thread t owns row t % R and chunks t / R + (256 / R) i, so a wave's
// loads walk 64 consecutive rows at one k.
template <int R>
struct StageAny {
  static constexpr int CH = R * 8 / NT;
  u32x4_t v[CH];

  __device__ __forceinline__ void load(const uint16_t* base, long long s_mn, long long s_k, int mn0, int mn_total,
                                       int k0, int K, int tid) {
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int row = tid % R;
      const int chunk = tid / R + (NT / R) * i;
      const int mn = mn0 + row, k = k0 + chunk * 8;
      // every load is issued, from an address clamped into the operand, and masked afterwards: no
      // branches, so the loads of a stage go out back to back and are awaited once (the mask is
      // arithmetic -- the sign of index - extent -- so that no select invites the compiler to put
      // the load back under a condition)
      const uint16_t* src = base + (long long)min(mn, mn_total - 1) * s_mn;
      const uint32_t row_mask = (uint32_t)((mn - mn_total) >> 31);
      uint32_t h[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int kc = min(k + j, K - 1);
        const uint32_t x = src[(long long)kc * s_k];
        h[j] = x & row_mask & (uint32_t)((k + j - K) >> 31);
      }
      v[i] = u32x4_t{h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)};
    }
  }

  __device__ __forceinline__ void store(unsigned char* lds, int tid) const {
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int row = tid % R;
      const int chunk = tid / R + (NT / R) * i;
      *reinterpret_cast<u32x4_t*>(lds + lds_off(row, chunk)) = v[i];
    }
  }
};

// staging modes of an operand: contiguous along mn / along k and aligned; the same two without
// the alignment; any strides
constexpr int MODE_MN = 0, MODE_K = 1, MODE_UMN = 2, MODE_UK = 3, MODE_ANY = 4;
template <int R, int MODE>
struct Stage;
template <int R>
struct Stage<R, MODE_K> : StageK<R, true> {};
template <int R>
struct Stage<R, MODE_MN> : StageMN<R, true> {};
template <int R>
struct Stage<R, MODE_UK> : StageK<R, false> {};
template <int R>
struct Stage<R, MODE_UMN> : StageMN<R, false> {};
template <int R>
struct Stage<R, MODE_ANY> : StageAny<R> {};

// XCD-aware remap of the linear workgroup id followed by a grouped tile order.
// Workgroups are handed to the 8 XCDs round-robin, so ids congruent mod 8 share an L2.  The
// remap gives each XCD a contiguous range of logical ids; the grouped order walks GROUP_M tile
// rows at a time so a contiguous range is a compact patch of the tile grid.
__device__ __forceinline__ void tile_coords(int wg, int tiles_m, int tiles_n, int* tm, int* tn) {
  const int nwg = tiles_m * tiles_n;
  constexpr int XCDS = 8;
  int logical = wg;
  if (nwg >= XCDS * 4) {
    const int per = (nwg + XCDS - 1) / XCDS;
    int tall = nwg % XCDS;
    if (tall == 0) tall = XCDS;
    const int xcd = wg % XCDS, local = wg / XCDS;
    logical = xcd < tall ? xcd * per + local : tall * per + (xcd - tall) * (per - 1) + local;
  }
  constexpr int GROUP_M = 8;
  const int per_group = GROUP_M * tiles_n;
  const int group = logical / per_group;
  const int first_m = group * GROUP_M;
  const int gsize = min(tiles_m - first_m, GROUP_M);
  const int in_group = logical - group * per_group;
  *tm = first_m + in_group % gsize;
  *tn = in_group / gsize;
}

template <typename T, int BM, int BN, int A_MODE, int B_MODE>
__global__ __launch_bounds__(NT) void gemm_mfma_kernel(GemmProblem p) {
  constexpr int WM = BM / 2, WN = BN / 2;  // wave tile
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int A_BYTES = BM * ROW_BYTES, B_BYTES = BN * ROW_BYTES;
  constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;

  const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  int tm, tn;
  tile_coords(blockIdx.x, tiles_m, tiles_n, &tm, &tn);
  const int m0 = tm * BM, n0 = tn * BN;
  const int bz = blockIdx.y;

  const uint16_t* A = (const uint16_t*)p.A + (long long)bz * p.sab;
  const uint16_t* B = (const uint16_t*)p.B + (long long)bz * p.sbb;

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  Stage<BM, A_MODE> sa;
  Stage<BN, B_MODE> sb;
  const int KT = (p.K + BK - 1) / BK;

  sa.load(A, p.sam, p.sak, m0, p.M, 0, p.K, tid);
  sb.load(B, p.sbn, p.sbk, n0, p.N, 0, p.K, tid);
  sa.store(lds, tid);
  sb.store(lds + A_BYTES, tid);
  __syncthreads();

  const int frow = lane & 31;
  const int fch = lane >> 5;

  for (int kt = 0; kt < KT; ++kt) {
    unsigned char* cur = lds + (kt & 1) * STAGE_BYTES;
    unsigned char* nxt = lds + ((kt + 1) & 1) * STAGE_BYTES;
    const bool more = kt + 1 < KT;
    if (more) {
      sa.load(A, p.sam, p.sak, m0, p.M, (kt + 1) * BK, p.K, tid);
      sb.load(B, p.sbn, p.sbk, n0, p.N, (kt + 1) * BK, p.K, tid);
    }
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      u32x4_t af[TM], bf[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        af[i] = *reinterpret_cast<const u32x4_t*>(cur + lds_off(wm0 + 32 * i + frow, 2 * kk + fch));
#pragma unroll
      for (int j = 0; j < TN; ++j)
        bf[j] = *reinterpret_cast<const u32x4_t*>(cur + A_BYTES + lds_off(wn0 + 32 * j + frow, 2 * kk + fch));
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = mfma32<T>(bf[j], af[i], acc[i][j]);   // B first: C^T tiles
    }
    if (more) {
      sa.store(nxt, tid);
      sb.store(nxt + A_BYTES, tid);
    }
    __syncthreads();
  }

  // epilogue: the MFMA took the B fragment first, so each 32 x 32 accumulator tile is C^T: a lane
  // holds row l % 32 and, per group of four registers, the four consecutive columns
  // 8 (v / 4) + 4 (l / 32) + 0..3 -- one 8-byte store per group where the row pitch and base of C
  // keep it aligned and the group lies inside N, element stores otherwise.
  Epilogue<T> ep(p);
  uint16_t* C = (uint16_t*)p.C + (long long)bz * p.scb;
  const bool wide = p.scn == 1 && (p.scm % 4) == 0 && (reinterpret_cast<uintptr_t>(C) & 7u) == 0;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + wm0 + 32 * i + (lane & 31);
    if (m >= p.M) continue;
    const float brow = ep.per_row ? ep.bias_at(m, 0) : 0.0f;
    uint16_t* crow = C + (long long)m * p.scm;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + wn0 + 32 * j + 8 * q + 4 * (lane >> 5);
        if (n >= p.N) continue;
        uint16_t h[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float bv = ep.per_row ? brow : (n + e < p.N ? ep.bias_at(0, n + e) : 0.0f);
          h[e] = ep.finish(acc[i][j][4 * q + e], bv);
        }
        if (wide && n + 3 < p.N) {
          uint2 w;
          w.x = (uint32_t)h[0] | ((uint32_t)h[1] << 16);
          w.y = (uint32_t)h[2] | ((uint32_t)h[3] << 16);
          *reinterpret_cast<uint2*>(crow + n) = w;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < p.N) crow[(long long)(n + e) * p.scn] = h[e];
        }
      }
    }
  }
}

// config ids: tile << 2 | a_kc << 1 | b_kc ; tile 1: 256x256, 2: 128x128, 3: 64x64
template <typename T, int BM, int BN, int A_MODE, int B_MODE>
hipError_t launch_one(const GemmProblem& p, hipStream_t stream) {
  constexpr size_t lds_bytes = 2 * (size_t)(BM + BN) * ROW_BYTES;
  auto kernel = gemm_mfma_kernel<T, BM, BN, A_MODE, B_MODE>;
  if (lds_bytes > 64 * 1024) {
    static std::atomic<uint32_t> configured{0};
    if (hipError_t e = ensure_lds_limit(reinterpret_cast<const void*>(kernel), (int)lds_bytes, configured); e != hipSuccess)
      return e;
  }
  const int tiles = ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
  hipLaunchKernelGGL(kernel, dim3(tiles, p.batch), dim3(NT), lds_bytes, stream, p);
  return launch_status(stream);
}

template <typename T, int BM, int BN>
hipError_t launch_layout(const GemmProblem& p, bool a_kc, bool b_kc, hipStream_t stream) {
  if (a_kc && b_kc) return launch_one<T, BM, BN, MODE_K, MODE_K>(p, stream);
  if (a_kc && !b_kc) return launch_one<T, BM, BN, MODE_K, MODE_MN>(p, stream);
  if (!a_kc && b_kc) return launch_one<T, BM, BN, MODE_MN, MODE_K>(p, stream);
  return launch_one<T, BM, BN, MODE_MN, MODE_MN>(p, stream);
}

// operands without the alignment guarantees: per operand, the unaligned form of the loader for
// its unit stride, or element-wise staging when it has none
template <typename T, int BM, int BN, int A_MODE>
hipError_t launch_any_b(const GemmProblem& p, hipStream_t stream) {
  if (p.sbk == 1) return launch_one<T, BM, BN, A_MODE, MODE_UK>(p, stream);
  if (p.sbn == 1) return launch_one<T, BM, BN, A_MODE, MODE_UMN>(p, stream);
  return launch_one<T, BM, BN, A_MODE, MODE_ANY>(p, stream);
}
template <typename T, int BM, int BN>
hipError_t launch_any_layout(const GemmProblem& p, hipStream_t stream) {
  if (p.sak == 1) return launch_any_b<T, BM, BN, MODE_UK>(p, stream);
  if (p.sam == 1) return launch_any_b<T, BM, BN, MODE_UMN>(p, stream);
  return launch_any_b<T, BM, BN, MODE_ANY>(p, stream);
}

template <typename T>
hipError_t launch_ring(const GemmProblem& p, bool a_kc, bool b_kc, hipStream_t stream);
template <>
hipError_t launch_ring<BF16>(const GemmProblem& p, bool a_kc, bool b_kc, hipStream_t stream) {
  if (a_kc && b_kc) return launch_ring_BF16_11(p, stream);
  if (a_kc) return launch_ring_BF16_10(p, stream);
  if (b_kc) return launch_ring_BF16_01(p, stream);
  return launch_ring_BF16_00(p, stream);
}
template <>
hipError_t launch_ring<F16>(const GemmProblem& p, bool a_kc, bool b_kc, hipStream_t stream) {
  if (a_kc && b_kc) return launch_ring_F16_11(p, stream);
  if (a_kc) return launch_ring_F16_10(p, stream);
  if (b_kc) return launch_ring_F16_01(p, stream);
  return launch_ring_F16_00(p, stream);
}

template <typename T>
hipError_t launch_m16(const GemmProblem& p, bool a_kc, bool b_kc, hipStream_t stream);
template <>
hipError_t launch_m16<BF16>(const GemmProblem& p, bool a_kc, bool b_kc, hipStream_t stream) {
  if (a_kc && b_kc) return launch_m16_BF16_11(p, stream);
  if (a_kc) return launch_m16_BF16_10(p, stream);
  if (b_kc) return launch_m16_BF16_01(p, stream);
  return launch_m16_BF16_00(p, stream);
}
template <>
hipError_t launch_m16<F16>(const GemmProblem& p, bool a_kc, bool b_kc, hipStream_t stream) {
  if (a_kc && b_kc) return launch_m16_F16_11(p, stream);
  if (a_kc) return launch_m16_F16_10(p, stream);
  if (b_kc) return launch_m16_F16_01(p, stream);
  return launch_m16_F16_00(p, stream);
}

// the 64-deep form of the 16x16x32 kernel
template <typename T>
hipError_t launch_m16d(const GemmProblem& p, bool a_kc, bool b_kc, hipStream_t stream) {
  if (T::dtype == srtReal16BF) {
    if (a_kc && b_kc) return launch_m16d_BF16_11(p, stream);
    if (a_kc) return launch_m16d_BF16_10(p, stream);
    if (b_kc) return launch_m16d_BF16_01(p, stream);
    return launch_m16d_BF16_00(p, stream);
  }
  if (a_kc && b_kc) return launch_m16d_F16_11(p, stream);
  if (a_kc) return launch_m16d_F16_10(p, stream);
  if (b_kc) return launch_m16d_F16_01(p, stream);
  return launch_m16d_F16_00(p, stream);
}

// the 128 x 256 form of the 16x16x32 ring kernel (k-contiguous A)
template <typename T>
hipError_t launch_m16d_partial(const GemmProblem& p, bool a_kc, bool b_kc, hipStream_t stream) {
  if (std::is_same<T, BF16>::value) {
    if (a_kc && b_kc) return launch_m16d_partial_BF16_11(p, stream);
    if (a_kc) return launch_m16d_partial_BF16_10(p, stream);
    if (b_kc) return launch_m16d_partial_BF16_01(p, stream);
    return launch_m16d_partial_BF16_00(p, stream);
  }
  if (a_kc && b_kc) return launch_m16d_partial_F16_11(p, stream);
  if (a_kc) return launch_m16d_partial_F16_10(p, stream);
  if (b_kc) return launch_m16d_partial_F16_01(p, stream);
  return launch_m16d_partial_F16_00(p, stream);
}

template <typename T>
hipError_t launch_m16d_tail(const GemmProblem& p, bool a_kc, bool b_kc, hipStream_t stream) {
  if (T::dtype == srtReal16BF) {
    if (a_kc && b_kc) return launch_m16d_tail_BF16_11(p, stream);
    if (a_kc) return launch_m16d_tail_BF16_10(p, stream);
    if (b_kc) return launch_m16d_tail_BF16_01(p, stream);
    return launch_m16d_tail_BF16_00(p, stream);
  }
  if (a_kc && b_kc) return launch_m16d_tail_F16_11(p, stream);
  if (a_kc) return launch_m16d_tail_F16_10(p, stream);
  if (b_kc) return launch_m16d_tail_F16_01(p, stream);
  return launch_m16d_tail_F16_00(p, stream);
}
// the split form of the 64-deep kernel: whole rounds of whole tiles, then one round of 192-wide ones
template <typename T>
hipError_t launch_m16d_split(const GemmProblem& p, bool a_kc, bool b_kc, hipStream_t stream) {
  if (T::dtype == srtReal16BF) {
    if (a_kc && b_kc) return launch_m16d_split_BF16_11(p, stream);
    if (a_kc) return launch_m16d_split_BF16_10(p, stream);
    if (b_kc) return launch_m16d_split_BF16_01(p, stream);
    return launch_m16d_split_BF16_00(p, stream);
  }
  if (a_kc && b_kc) return launch_m16d_split_F16_11(p, stream);
  if (a_kc) return launch_m16d_split_F16_10(p, stream);
  if (b_kc) return launch_m16d_split_F16_01(p, stream);
  return launch_m16d_split_F16_00(p, stream);
}
// the 128 x 256 half tile of the 64-deep kernel (k-contiguous A)
template <typename T>
hipError_t launch_m16dh(const GemmProblem& p, bool b_kc, hipStream_t stream) {
  if (T::dtype == srtReal16BF) return b_kc ? launch_m16dh_BF16_11(p, stream) : launch_m16dh_BF16_10(p, stream);
  return b_kc ? launch_m16dh_F16_11(p, stream) : launch_m16dh_F16_10(p, stream);
}
// the 256 x 128 half tile of the 64-deep kernel (A not k-contiguous)
template <typename T>
hipError_t launch_m16dn(const GemmProblem& p, bool b_kc, hipStream_t stream) {
  if (T::dtype == srtReal16BF) return b_kc ? launch_m16dn_BF16_01(p, stream) : launch_m16dn_BF16_00(p, stream);
  return b_kc ? launch_m16dn_F16_01(p, stream) : launch_m16dn_F16_00(p, stream);
}
// the 128 x 128 quarter tile of the 16x16x32 kernel (128-deep units), all four layouts
template <typename T>
hipError_t launch_m16q(const GemmProblem& p, bool a_kc, bool b_kc, hipStream_t stream) {
  if (T::dtype == srtReal16BF) {
    if (a_kc) return b_kc ? launch_m16q_BF16_11(p, stream) : launch_m16q_BF16_10(p, stream);
    return b_kc ? launch_m16q_BF16_01(p, stream) : launch_m16q_BF16_00(p, stream);
  }
  if (a_kc) return b_kc ? launch_m16q_F16_11(p, stream) : launch_m16q_F16_10(p, stream);
  return b_kc ? launch_m16q_F16_01(p, stream) : launch_m16q_F16_00(p, stream);
}
template <typename T>
hipError_t launch_m16h(const GemmProblem& p, bool b_kc, hipStream_t stream) {
  if (T::dtype == srtReal16BF) return b_kc ? launch_m16h_BF16_11(p, stream) : launch_m16h_BF16_10(p, stream);
  return b_kc ? launch_m16h_F16_11(p, stream) : launch_m16h_F16_10(p, stream);
}

// tile 1 (256 x 256) is the ring kernel, tile 5 the same ring on 16x16x32 MFMAs, tile 6 its 128 x 256
// form; tiles 2 and 3 are the register-staged kernels above, 7 and 8 the same without alignment rules
template <typename T>
hipError_t launch_tile(const GemmProblem& p, int tile, bool a_kc, bool b_kc, hipStream_t stream) {
  switch (tile) {
    case 1: return launch_ring<T>(p, a_kc, b_kc, stream);
    case 4: return T::dtype == srtReal16BF ? launch_kc64_BF16(p, stream) : launch_kc64_F16(p, stream);
    case 5: return launch_m16<T>(p, a_kc, b_kc, stream);
    case 6: return launch_m16h<T>(p, b_kc, stream);
    case 9: return launch_m16d<T>(p, a_kc, b_kc, stream);
    case 10: return launch_m16d_tail<T>(p, a_kc, b_kc, stream);
    case 11: return launch_m16d_split<T>(p, a_kc, b_kc, stream);
    case 12: return launch_m16dh<T>(p, b_kc, stream);
    case 13: return launch_m16dn<T>(p, b_kc, stream);
    case 14: return launch_m16q<T>(p, a_kc, b_kc, stream);
    case 2: return launch_layout<T, 128, 128>(p, a_kc, b_kc, stream);
    case 7: return launch_any_layout<T, 128, 128>(p, stream);
    case 8: return launch_any_layout<T, 64, 64>(p, stream);
    default: return launch_layout<T, 64, 64>(p, a_kc, b_kc, stream);
  }
}

inline bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

}  // namespace

// The MFMA family needs: a 16-bit element type, C rows contiguous, each operand contiguous
// along k or along its other dimension with 16-byte aligned rows, and extents along the
// contiguous dimensions that are multiples of 8 (so every 16-byte load is whole).
// Layout bits of a qualifying problem (bit 1: A k-contiguous, bit 0: B k-contiguous), or -1.
static int mfma_layout(const GemmProblem& p) {
  if (p.dtype != srtReal16BF && p.dtype != srtReal16F) return -1;
  if (p.scn != 1 || p.K < 1) return -1;
  if (p.batch > 65535) return -1;
  bool a_kc, b_kc;
  if (p.sak == 1 && (p.K % 8) == 0) a_kc = true;
  else if (p.sam == 1 && (p.M % 8) == 0) a_kc = false;
  else return -1;
  if (p.sbk == 1 && (p.K % 8) == 0) b_kc = true;
  else if (p.sbn == 1 && (p.N % 8) == 0) b_kc = false;
  else return -1;
  const long long lda = a_kc ? p.sam : p.sak, ldb = b_kc ? p.sbn : p.sbk;
  // a single row/column operand may carry any leading stride; otherwise rows must stay aligned
  if ((lda % 8) != 0 || (ldb % 8) != 0) return -1;
  if ((p.sab % 8) != 0 || (p.sbb % 8) != 0) return -1;
  if (!aligned16(p.A) || !aligned16(p.B)) return -1;
  if (p.sam < 0 || p.sak < 0 || p.sbk < 0 || p.sbn < 0 || p.scm < 0) return -1;
  return (a_kc ? 2 : 0) | (b_kc ? 1 : 0);
}

// Configuration for a given tile (1: 256 x 256 ring, 2: 128 x 128, 3: 64 x 64, 4: 256 x 256 with
// 64-deep stages for two k-contiguous operands, 5: the 256 x 256 ring on 16x16x32 MFMAs, 6: its
// 128 x 256 form for a k-contiguous A, 9: the 16x16x32 kernel with 64-deep staging units), or 0 when the
// problem does not qualify for it.  10: tile 9's tail-sharing form.  11: its split form (a last round of 192-wide tiles).  12: its 128 x 256 half tile (k-contiguous A).  13: its 256 x 128 half tile (A not k-contiguous).
// 14: the 128 x 128 quarter tile on 128-deep units (any layout).
int mfma_config(const GemmProblem& p, int tile) {
  if (tile == 7 || tile == 8) {   // any strides and alignment (the loaders are chosen at launch)
    if (p.dtype != srtReal16BF && p.dtype != srtReal16F) return 0;
    if (p.K < 1 || p.batch > 65535) return 0;
    return tile << 2;
  }
  const int layout = mfma_layout(p);
  if (layout < 0 || tile < 1 || (tile > 6 && (tile < 9 || tile > 14))) return 0;
  if ((tile == 1 || tile >= 4) && !ring_fits_problem(p, (layout & 2) != 0, (layout & 1) != 0)) return 0;
  if ((tile == 9 || tile == 12 || tile == 13) && !(p.K % 64 == 0 && p.K >= 256)) return 0;   // whole 64-deep units, at least four
  if (tile == 14 && !(p.K % 128 == 0 && p.K >= 256)) return 0;   // whole 128-deep units, at least two
  if (tile == 10) {   // left-over tiles to share, k in whole quads, no transcendental activation
    const bool trans = p.activation == srtActivationSigmoid || p.activation == srtActivationTanh || p.activation == srtActivationElu;
    if (trans || !m16d_tail_fits_BF16_xx(p)) return 0;
  }
  // whole rounds of whole tiles and a last round that 192-wide tiles fill, no transcendental activation (pinned or tuned plans only)
  if (tile == 11 && !m16d_split_fits_BF16_xx(p)) return 0;
  if ((tile == 6 || tile == 12) && (layout & 2) == 0) return 0;   // the 128-row A region is k-contiguous
  if (tile == 13 && (layout & 2) != 0) return 0;                  // the 256 x 128 half tile is for the other A layouts
  if (tile == 4 && layout != 3) return 0;   // the 64-deep kernel takes two k-contiguous operands only
  return (tile << 2) | layout;
}

int mfma_splitk_parts(const GemmProblem& p);

// Whether the 256 x 128 half tile of an A that is not k-contiguous is the choice: when one round of them holds the problem
// (whole tiles would leave half of those compute units idle) and the k loop is short enough that cutting it does not do better.
//   K <= 1024       always: 512 x 512 x 512 x^T . W 10.7 us against 15.2 for 64 x 64 tiles, 512 x 2048 x 1024 15.9 against 22.6
//                   whole, 512 x 512 x 1024 15.8 against 20.4 for split-K; x^T . W^T 1024 x 1024 x 1024 15.9 against 20.0 (64 x 64)
//   K <= 2048       from 64 of them: 2048^3 26.5 us against 32.0 shared and 38.9 whole; 2048 x 4096 x 2048 32.5 against 39;
//                   1024 x 2048 x 2048 26.0 against 27.8 for split-K
//   K = 4096        x^T . W^T only (a k-contiguous B is staged without waste), from 96: 2048 x 2048 x 4096 45.0 us against
//                   49.5 shared, 1536 x 4096 x 4096 47.2 against 51.2; x^T . W 1024 x 4096 x 4096: 46.0 against 42.9 shared
static bool narrow_round(const GemmProblem& p, int layout) {
  // (from 64 rows and columns: a batch of 64 x 512 x 1024 problems runs 16.2 us in these tiles, three quarters padding,
  // against 22.6 in whole tiles and 19.4 in 64 x 64 ones; 4 x 128 x 128 x 1024: 15.6 against 22.4)
  if (layout < 0 || (layout & 2) != 0 || mfma_config(p, 13) == 0 || p.M < 64 || p.N < 64) return false;
  const long long tn = (long long)((p.M + 255) / 256) * ((p.N + 127) / 128) * p.batch;
  if (tn > compute_units()) return false;
  if (p.K > 2048) {
    // (a batch at K = 4096: only tiles that are mostly padding rows, and only a device's worth of them -- 64 x 64 x 512 x 4096
    // x^T . W^T 68.4 us against 83.3 shared and 97.7 whole; 16 x 512 x 512 x 4096: 60.5 against 54.9 shared; 16 x 64 x 512 x 4096,
    // 64 tiles: 43.2 against 39.3 shared)
    if (p.batch > 1) return layout == 1 && p.K < 8192 && p.M <= 128 && 2 * tn > compute_units();
    // (with fewer rows four parts of the k loop do better when K can be cut in four: 384 x 6144 x 4096 36.0 us in parts against
    // 43.4; 192 x 12568 x 3264, which only halves: 36.0 against 41.7)
    // (x^T . W only where the k extent is not in whole quads of 64-deep units, so that no tiles can be shared: 1048 x 6392 x 3456
    // 49.8 us against 61.2 whole)
    return (layout == 1 || p.K % 256 != 0) && p.K < 8192 && tn >= 96 && (p.M >= 1024 || mfma_splitk_parts(p) < 4);
  }
  // (tiles that are three quarters padding rows only while they leave half the device free: 64 x 64 x 512 x 1024, 256 of them,
  // 27.1 us against 23.1 in 128 whole tiles)
  if (p.M <= 64 && 2 * tn > compute_units()) return false;
  if (p.K <= 1024) return true;
  return tn >= 64;
}

int mfma_select(const GemmProblem& p) {
  const int layout = mfma_layout(p);
  auto tiles = [&](int t) { return (long long)((p.M + t - 1) / t) * ((p.N + t - 1) / t) * p.batch; };
  // the device's compute units and half of them: "a device's worth" and "half a device's worth" of tiles below (the
  // other tile counts in the rules are measured cross-over points on a 256-unit device)
  const long long cus = compute_units(), half_cus = cus / 2;
  // operands that miss the alignment rules: unaligned or element-wise staging, 128 x 128 tiles once they fill the device
  if (layout < 0) return mfma_config(p, tiles(128) >= cus ? 7 : 8);
  // Tile choice, from measurements over mid-size problems (1024^3 .. 4096 x 14336 x 4096):
  //  * the 256 x 256 kernels are so much more efficient per tile (deep prefetch, 4x the arithmetic
  //    intensity) that they win long before they can fill the device: from 24 tiles up (48 when K < 1024) for the
  //    ring kernel (3072^3, 144 tiles: 64 us against 143 us with 128 x 128 tiles);
  //  * with both operands k-contiguous the 64 x 64 kernel reads whole lines too and stays ahead up
  //    to about 96 tiles of 256 x 256 (2048^3 NT: 36 us against 44 us); from there the ring kernel
  //    runs until the device is three quarters full (2048 x 4096 x 4096 NT, 128 tiles: 84 us
  //    against 88 us) and then the 64-deep 256 x 256 kernel takes over (whole-line loads where
  //    the ring kernel moves half lines: 4096^3 NT 114 us against 126 us, 8192^3 NT 1351 against
  //    1336 TFLOP/s);
  //  * once the device is half full and the k loop is long, sustained speed is set by the power
  //    limit, and the 16x16x32 form of the ring kernel, cheaper per flop, wins in every layout
  //    (8192^3: 1410-1490 against 1340-1390 TFLOP/s; 4096 x 11008 x 4096: 280 us against
  //    298-308 us; 3072^3, 144 tiles: 68 us against 71 us; 2048 x 4096 x 4096, 128 tiles: 84 us
  //    against 85 us).  Its loop has less slack per MFMA, so where clocks are not the limit -- a
  //    partly filled device -- the 32x32x16 kernels stay ahead (2048^3: 42 us against 43.5 us;
  //    1024 x 4096 x 4096: 73 us against 77 us), and with short k loops (K = 1024) nothing
  //    separates them;
  //  * below those thresholds every CU should get a workgroup: 64 x 64 tiles (batch 32 x 256^3:
  //    7.7 us against 15.0 us with 128 x 128).  128 x 128 is kept for problems that do not meet
  //    the 256 x 256 kernels' preconditions but have at least one such tile per CU.
  const bool big_ok = ring_fits_problem(p, (layout & 2) != 0, (layout & 1) != 0);
  const long long t256 = tiles(256);
  //  * with a k-contiguous A the 16x16x32 kernel also comes with 128 x 256 tiles: twice the
  //    workgroups, which is what a problem that leaves compute units idle needs (2048^3: 29 us
  //    against 42 us; 512 x 14336 x 4096: 59 against 82; 256 x 1024 x 1024: 15 against 19 for 64 x 64
  //    tiles).  On a full device a half tile costs about 0.6 of a whole one (4096^3: 129 us
  //    against 105 us), so the choice goes by rounds of the persistent grid: half tiles when
  //    0.6 x their rounds does not exceed the whole tiles' rounds -- always when they fit in one
  //    round (2048 x 4096 x 2048: 35 us against 47 us), and where whole tiles quantise badly
  //    (1536 x 11008 x 4096, 258 tiles: 152 us against 171 us; 3072 x 3072 x 1024, 144 tiles
  //    against 288 halves: 28 us whole, 32.5 us halves).  With a k-contiguous B as well the half
  //    tile is dearer (0.68: both operands arrive as half cache lines), so there it is taken only
  //    when it fits in one round (1536 x 11008 x 4096 NT: 190 us against 168 us whole), and the
  //    64 x 64 kernel is as good up to about 96 half tiles (1024 x 1024 x 2048: 20 us against 23 us).
  const long long th = (long long)((p.M + 127) / 128) * ((p.N + 255) / 256) * p.batch;
  const long long rounds256 = (t256 + cus - 1) / cus, rounds_h = (th + cus - 1) / cus;
  //  * a problem of a handful of tiles is bound by the latency of its k stages, and the ring's
  //    deep prefetch beats the 64 x 64 kernel's load-wait-compute stages even on one or two
  //    workgroups (192 x 128 x 128: 6.5 us against 8.0 us; 96 x 128 x 768: 12.5 against 14.7);
  //    the same holds for short k loops on many tiles, where the 64 x 64 kernel's 8-byte stores
  //    of the result also count (512 x 16384 x 128: 9.0 us against 18.3 us; 3072 x 11008 x 64
  //    with A m-contiguous, whole tiles: 27 us against 71 us);
  //  * a whole 256 x 256 tile is half padding or more with up to 128 rows or columns: there the
  //    64 x 64 kernel wins (48 x 16384 x 768 with A m-contiguous: 15.9 us against 20.5 us;
  //    128 x 14336 x 128: 8.0 against 10.2);
  //  * on a device at least half full the 16x16x32 ring is ahead of the 32x32x16 one for short
  //    k loops too (3072 x 8192 x 1024 with A m-contiguous: 56 us against 65 us; 3072 x 16384 x 512:
  //    60 against 67; 4096 x 4096 x 1024: 34.6 against 36.2) -- except with two k-contiguous
  //    operands, where the 64-deep kernel keeps short k loops (8192 x 8192 x 1024: 138 us against 146).
  // Half tiles: with 64 columns or fewer only for longer k loops and an n-contiguous B (1536 x 64 x 128:
  // 10.4 us against 6.7 us for 64 x 64 tiles, 1536 x 64 x 768: 12.8 against 15.1; 32 x 1024 x 64 x 4096
  // with B k-contiguous: 97 against 67).  With two k-contiguous operands they are taken only in one round (8 x 128 x
  // 4096 x 1024: 21 us against 28 us; 8 x 512 x 2048 x 256: 10.5 against 14.0), by the counts below.
  // (from 72 half tiles in one round: 1536 x 1536 x 1024 x . W^T, 72 of them: 14.8 us against 16.8 for 64 x 64 tiles;
  // 1024 x 2048 x 2048, 64 of them: 25.7 against 22.9)
  // (a batch goes by the same count: 64 x 256 x 256 x 1024, 128 half tiles: 20.4 us against 31.9 for 64 x 64 tiles; 16 x 128 x
  // 128 x 1024, 16 of them: 14.2 against 12.0; 64 x 256 x 1024 x 256, 512 of them: 27.4 against 18.4 for whole tiles;
  // with 64 rows or fewer half of a half tile is padding: 64 x 64 x 512 x 256 9.3 against 8.2)
  // (a batch of 128 whole tiles or more stays whole: its tiles share no operand, and the half tile's lower arithmetic
  // intensity shows -- 16 x 640 x 640 x 8192: 264 us against 169-174)
  // (a last row of half tiles that is mostly padding: 169 x 9824 x 504, 78 half tiles, 11.1 us against 9.8 for 64 x 64; up to
  // a quarter of padding is fine: 664 x 7536 x 352 10.2 us against 16.3.  A long k loop wants more of the device: 5 x 1020 x
  // 408 x 3368, 80 half tiles, 70 us against 44 for 64 x 64 tiles.  With 128 rows or fewer whole tiles are no alternative, and
  // a short k loop is all stores: half tiles whatever the rounds, 45 x 72 x 2240 x 64 10.4 us against 18.3)
  const long long m_pad = (p.M + 127) / 128 * 128;
  const bool half_fill_ok = 4 * (m_pad - p.M) <= m_pad;
  // (3205 x 984 x 3800, 104 half tiles: 48 us against 56; short rows with k loops from 1024: 3 x 194 x 3080 x 1672, 78 half
  // tiles, 38 us against 25 for 64 x 64 tiles)
  // (those two are of batches; a single matrix shares its operands between tiles and takes half tiles from 72: 397 x 7528 x
  // 1056, 120 of them, 15 us against 21; 664 x 3208 x 8544, 78, 87 against 97)
  // (a batch in the 64-deep half tile, whose loads move whole lines of both operands, from 64 of them whatever K, and with
  // rows that are half padding: 16 x 384 x 384 x 1024, 96 half tiles, 16.0 us against 19.7 for 64 x 64 tiles; 64 x 128 x 128 x
  // 4096, 64 of them, 43.2 against 58.0; 64 x 64 x 512 x 1024, 128 of them half empty, 18.6 against 23.0)
  // (not for short k loops: 32 x 256 x 256 x 256 7.7 us against 7.1 for 64 x 64 tiles, 64 x 128 x 128 x 256 7.7 against 6.9)
  const bool deep_batch = p.batch > 1 && p.K % 64 == 0 && p.K >= 1024;
  const long long th_min = deep_batch ? 64 : p.batch == 1 ? 72 : p.K >= 2048 ? 96 : (p.K >= 1024 && p.M < 512) ? 128 : 72;
  const bool fill_ok = half_fill_ok || (deep_batch && 2 * (m_pad - p.M) <= m_pad);
  const bool one_round = th >= th_min && rounds_h == 1 && fill_ok && (p.batch == 1 || t256 < half_cus || (deep_batch && t256 == half_cus));
  const bool small_rows = p.M <= 128 && p.K <= 512 && th >= 72;
  // (x . W^T with a short k loop and whole tiles that leave a second or later round at most half full: twice the
  // workgroups fill it better -- 3072 x 6144 x 512, 288 tiles: 25.4 us against 27.3 whole; 3072 x 6144 x 256: 18.7 against
  // 20.7; 3072 x 6144 x 1024: 39.7 against 42.8.  Whole rounds stay whole: 4096 x 4096 x 512 19.8 us against 21.4)
  const bool short_nt = p.K <= 1024 && p.K % 64 == 0 && p.K >= 256 && t256 > cus && t256 % cus != 0 && 2 * (t256 % cus) <= cus &&
                        p.batch == 1 && half_fill_ok;
  const bool half_nt = (p.M > 64 || (deep_batch && p.M == 64)) && (one_round || small_rows || short_nt);
  // (a round of half tiles takes 0.6 of a round of whole ones on the 32-deep kernels, 0.7 against the 64-deep
  // one: 4096 x 10240 x 4096, five rounds of half tiles against three of whole ones, 265 us against 249 us)
  const bool deep = p.K % 64 == 0 && p.K >= 512;
  const bool half_ok = p.K >= 64 && (p.N > 64 || (layout == 2 && p.K >= 512)) &&
                       (layout == 3 ? half_nt : (deep ? 7 : 6) * rounds_h <= 10 * rounds256);
  // Whole tiles: padding up to 256 rows and columns is affordable when the alternative is the 64 x 64
  // kernel on two n- / m-contiguous operands, which it transposes in registers, and the device is at
  // least half full (64 x 8 x 1024 x 256: 13.6 us against 19.6 us), or when the k loop is long, where the
  // ring's prefetch outruns the 64 x 64 kernel's load-wait-compute stages whatever the tile count
  // (16 x 128 x 2048 x 2048: 45 us against 110 us; 8 x 32 x 128 x 4096: 72 against 82; at K = 2048 with a
  // k-contiguous B the 64 x 64 kernel is still ahead: 8 x 512 x 64 x 2048 34 us against 39 us).  With a
  // short k loop and few tiles, or a k-contiguous B and under 128 rows, it is not (48 x 16384 x 768: 20.5 us
  // against 15.9 us for 64 x 64 tiles; 128 x 14336 x 128: 10.2 against 8.0; 8 x 32 x 4096 x 64: 8.6 against
  // 6.6; but 64 x 128 x 1024 x 128: 12.3 against 18.5).
  // (an A that is not k-contiguous has no half tiles and the 64 x 64 kernel's k loop is slow on it: from K = 1024 whole
  // tiles even when most of their rows are padding -- 64 x 128 x 128 x 1024 with A m-contiguous 22.6 us against 30.9,
  // 64 x 64 x 512 x 1024 22.7 against 28.4)
  const bool whole_ok = big_ok && ((p.M > 128 && p.N > 128) || p.K >= 4096 ||
                                   ((layout & 2) == 0 && p.K >= (p.batch > 1 ? 512 : 1024) && p.M >= 64 && p.N >= 64) ||
                                   (layout == 0 && p.K >= 512) ||   // (8 x 88 x 2576, one tile: 51 us against 63; 16 x 2560 x 960: 22 against 25)
                                   (t256 >= half_cus && (layout == 0 || p.K >= 2048 || (p.M >= 72 && p.N >= 72))));
  // (a device's worth of tiles that are two thirds padding still beats 64 x 64 tiles: 41 x 1480 x 72 x 1248 x . W^T 37 us
  // against 68, 21 x 1840 x 88 x 152 11 against 17; not with a handful of rows: 35 x 8 x 2024 x 1144 52 against 38)
  // (with neither operand k-contiguous the 64 x 64 kernel transposes both in registers: whole tiles from 12 up,
  // 512 x 1536 x 1024: 22.7 us against 24.9)
  // (x^T . W^T at K = 1024: a single matrix of 16-32 tiles is 6-10 % faster in 64 x 64 tiles -- 1024 x 2048 x 1024 20.9 us
  // against 22.8 --, a batch, whose tiles share no operand, in whole ones from 16: 16 x 256 x 256 x 1024 21.9 against 24.3)
  const long long ring_from = layout == 3 ? 96
                            // (312 x 6136 x 80, 48 tiles: 9.9 us against 8.7; at K = 256 the 64-deep kernel is ahead from 36 tiles:
                            // 1536 x 1536 x 256 11.3 us against 12.1, 1024 x 3072 x 256 11.5 against 12.6)
                            : layout == 0 ? (p.K >= 1024 ? 1 : p.K >= 512 ? 8 : p.K >= 256 ? 32 : 48)   // (888 x 3616 x 176, 60 tiles: 11.6 us against 17.1 in 64 x 64 tiles)
                            : p.K < 1024 ? 32 : layout == 1 ? (p.batch > 1 ? 16 : 40) : 24;
  //  * the 64-deep form of the 16x16x32 kernel (whole-line loads of k-contiguous operands, one barrier per 128
  //    MFMAs) is ahead of the 32-deep one in every layout once the device is half full (8192^3, same run:
  //    NN 1440 -> 1505 TFLOP/s, NT 1420 -> 1531, TN 1443 -> 1501, TT 1477 -> 1538), and of the 32x32x16
  //    64-deep kernel that two k-contiguous operands used to take for short k loops; it needs whole units
  //    (K a multiple of 64, at least 512).  With an A that is not k-contiguous -- no half tiles -- it also takes
  //    over from the 32x32x16 ring below half a device (2048 x 3072 x 1024, 96 tiles: 23-24 us against 26; 2048 x
  //    2048 x 2048, 64 tiles: 38-40 against 40-41; 1024 x 2048 x 1024, 32 tiles: 23 against 25)
  //    Four units (K = 256) are enough: 2048 x 3072 x 256 with A m-contiguous 11.8 us against 12.8-13.8 for the
  //    32-deep kernels, 3072 x 8192 x 256 x . W^T 21.3 against 24.7.
  const bool deep_ok = p.K % 64 == 0 && p.K >= 256;
  // an m-contiguous A against a k-contiguous B, a short k loop and under 64 tiles: the 64 x 64 kernel (1024 x 2048
  // x 256: 9.6 us against 12.4 for whole tiles; 512 x 4096 x 512: 13.2 against 15.0; at 64 tiles whole tiles win)
  // (a single matrix: the tiles of a batch share no operand and whole tiles win there -- 48 x 256 x 256 x 512: 14.7 us
  // against 19.4)
  const bool small_tt = layout == 1 && p.K <= 512 && t256 < 64 && p.batch == 1;
  // two k-contiguous operands and a last row of tiles that is half padding or more: the 32x32x16 64-deep kernel loses
  // less to the padding (64 x 384 x 384 x 4096: 130 us against 155 for the 16x16x32 one, K = 256: 14.9 against 16.9)
  const int m_rest = p.M % 256;
  const bool padded_nt = layout == 3 && m_rest >= 1 && m_rest <= 128 && p.M < 1024 && t256 >= half_cus;
  int tile;
  // (half tiles in their 64-deep form whenever K allows: never behind the 32-deep one, 2-5 % ahead for x . W -- 2048^3 26.1 ->
  // 24.9 us -- and 10-17 % for x . W^T, whose loads then move whole lines: 2048 x 4096 x 2048 34.1 -> 28.2 us)
  // (an A that is not k-contiguous has its half tile too, 256 x 128: taken when one round holds the problem, which whole
  // tiles would leave half empty -- see narrow_round for the measured pairs; with K = 4096 or more the shared tiles and
  // split-K, asked earlier, keep what they took: 1024 x 4096 x 4096 42.9 us shared against 46.0)
  if (narrow_round(p, layout)) tile = 13;
  else if (big_ok && (layout & 2) != 0 && half_ok) tile = deep_ok ? 12 : 6;
  else if (whole_ok && padded_nt) tile = 4;
  else if (small_tt) tile = 3;
  else if (whole_ok && deep_ok && (t256 >= half_cus || ((layout & 2) == 0 && t256 >= ring_from))) tile = 9;
  // (two k-contiguous operands and a k extent that is not a whole number of 32-deep stages: the 16x16x32 ring loses its
  // prefetch across tiles there, 4826 x 12408 x 7056: 833 us against 703 for the 32x32x16 64-deep kernel)
  else if (whole_ok && layout == 3 && t256 >= half_cus && p.K % 32 != 0) tile = 4;
  else if (whole_ok && t256 >= half_cus && (layout != 3 || p.K >= 2048)) tile = 5;
  else if (whole_ok && layout == 3 && t256 >= half_cus) tile = 4;   // (1480 x 7920 x 128, 186 tiles: 11.8 us against 14.2 for the ring)
  // (k loops too short for the 64-deep kernel, A not k-contiguous: the 16x16x32 ring, 4 x 1024 x 1024 x 64: 9.1 us against 10.1)
  else if (whole_ok && !deep_ok && (layout & 2) == 0 && t256 >= ring_from && mfma_config(p, 5) != 0) tile = 5;
  // (a handful of rows against a k-contiguous B: the 64 x 64 tiles, 4 x 8 x 104 x 7264 103 us against 116)
  else if (whole_ok && (t256 >= ring_from || (p.K >= 4096 && (layout == 0 || (layout == 1 && p.M > 64))))) tile = 1;
  else if (!big_ok && tiles(128) >= cus) tile = 2;
  else tile = 3;
  return (tile << 2) | layout;
}

// ---- split-K over the 256 x 256 kernel ----------------------------------------------------------
// A problem with few 256 x 256 tiles and a long k loop leaves most compute units idle.  Its k range
// is cut into S equal parts that run as S "batches" of the 16x16x32 ring kernel (operand batch
// stride = one part's k extent), each writing its fp32 accumulators to a workspace [S][M][N]; a
// second kernel adds the parts in a fixed order and applies bias, activation and the one rounding.
// The sums are fp32 throughout, and the result does not depend on timing.
namespace {

template <typename T>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* part, int parts, GemmProblem p) {
  using S = typename T::storage;
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  const int n8 = p.N / 8;   // 8 columns per lane
  const long long id = (long long)blockIdx.x * 256 + threadIdx.x;
  if (id >= (long long)p.M * n8) return;
  const int m = (int)(id / n8), n = (int)(id - (long long)m * n8) * 8;
  const long long mn = (long long)p.M * p.N;
  const float* src = part + (long long)m * p.N + n;
  f32x4 lo = {0.0f, 0.0f, 0.0f, 0.0f}, hi = lo;
  for (int s = 0; s < parts; ++s) {
    lo += *reinterpret_cast<const f32x4*>(src + s * mn);
    hi += *reinterpret_cast<const f32x4*>(src + s * mn + 4);
  }
  Epilogue<T> ep(p);
  union { S h[8]; uint4 v; } out;
#pragma unroll
  for (int e = 0; e < 8; ++e) out.h[e] = ep.finish(e < 4 ? lo[e] : hi[e - 4], ep.bias_at(m, n + e));
  *reinterpret_cast<uint4*>((S*)p.C + (long long)m * p.scm + n) = out.v;
}

template <typename T>
hipError_t launch_m16_partial(const GemmProblem& p, bool a_kc, bool b_kc, hipStream_t stream);
template <>
hipError_t launch_m16_partial<BF16>(const GemmProblem& p, bool a_kc, bool b_kc, hipStream_t stream) {
  if (a_kc && b_kc) return launch_m16_partial_BF16_11(p, stream);
  if (a_kc) return launch_m16_partial_BF16_10(p, stream);
  if (b_kc) return launch_m16_partial_BF16_01(p, stream);
  return launch_m16_partial_BF16_00(p, stream);
}
template <>
hipError_t launch_m16_partial<F16>(const GemmProblem& p, bool a_kc, bool b_kc, hipStream_t stream) {
  if (a_kc && b_kc) return launch_m16_partial_F16_11(p, stream);
  if (a_kc) return launch_m16_partial_F16_10(p, stream);
  if (b_kc) return launch_m16_partial_F16_01(p, stream);
  return launch_m16_partial_F16_00(p, stream);
}

}  // namespace

// Number of k parts for the split-K plan, or 0 when the problem does not qualify: one batch,
// the 256 x 256 kernel's preconditions, parts of equal length that are whole k stages and at least
// 16 of them (512 k), and no more parts than it takes to give every compute unit a tile.
int mfma_splitk_parts(const GemmProblem& p) {
  const int layout = mfma_layout(p);
  if (layout < 0 || p.batch != 1) return 0;
  if (!ring_fits_problem(p, (layout & 2) != 0, (layout & 1) != 0)) return 0;
  if ((reinterpret_cast<uintptr_t>(p.C) & 15u) != 0 || (p.scm % 8) != 0) return 0;
  // a k-contiguous A of at most 128 rows runs the pass on 128 x 256 tiles (half the padding to multiply)
  const long long t256 = (long long)((p.M + 255) / 256) * ((p.N + 255) / 256);   // also the count of half tiles then
  int parts = 0;
  for (int s = 2; s <= 16; s *= 2) {
    if (t256 * s > compute_units()) break;
    if (p.K % (s * 32) != 0 || p.K / s < 512) break;
    parts = s;
  }
  return parts;
}

// Whether the heuristic takes the split-K plan.  The fp32 parts cost a fixed 25-30 us to write and
// add up (about 67 MB each way whatever the shape), and with a k-contiguous A the 128 x 256 tiles
// already double the workgroups at no such cost, so the split must buy more than that:
//   A not k-contiguous      four parts from K = 2048 (256 x 2048 x 2048 TN: 27 us against 45 us for
//                           64 x 64 tiles), two from K = 4096 (2048 x 4096 x 4096 TN: 77 us against
//                           87 us; at K = 2048 two parts lose, 1024 x 8192 x 2048: 56 against 47)
//   A k-contiguous, M <= 128  the same rule (the pass runs on 128 x 256 tiles: 64 x 2048 x 2048: 18 us
//                           against 25 us for half tiles alone; 64 x 14336 x 4096: 32 us against 46 us)
//   A and B k-contiguous    four parts from K = 4096 (768 x 4096 x 4096: 47 us against 52 us for half
//                           tiles), two from K = 8192 (1536 x 4096 x 11008: 136 us against 168 us)
//   A k-, B n-contiguous    eight parts from K = 4096 (512 x 4096 x 4096: 43 us against ~50 us for half
//                           tiles; with four parts the two tie), four from K = 8192 (2048 x 2048 x
//                           8192: 79 us) or when M <= 192 (64 x 14336 x 4096: 37 us against 46 us;
//                           256 x 14336 x 4096: 54 us against 47 us for half tiles);
//                           two parts lose to half tiles (2048 x 4096 x 11008: 183 against 154)
bool mfma_prefers_splitk(const GemmProblem& p) {
  const int parts = mfma_splitk_parts(p);
  if (parts < 2) return false;
  const int layout = mfma_layout(p);
  // an A that is not k-contiguous and one round of its 256 x 128 half tiles: those do better than the parts (narrow_round)
  if (narrow_round(p, layout)) return false;
  // a handful of tiles: nothing else occupies the device (192 x 512 x 2048: 23 us against 32 us for
  // 64 x 64 tiles; 512 x 512 x 3072: 28 us against 35 us for half tiles; with both operands
  // k-contiguous the 64 x 64 kernel holds out longer -- 192 x 512 x 2048: 19 us against 22 us, but
  // 3072 x 128 x 3072: 33 us against 28 us)
  const long long t256 = (long long)((p.M + 255) / 256) * ((p.N + 255) / 256);
  // (a k-contiguous A has half tiles: 1024 x 1536 x 2048, 24 tiles: 25.5 us in half tiles against 27.9 in four parts;
  // with neither operand k-contiguous even two parts of a handful of tiles pay: 512 x 512 x 1024: 20 us against 25)
  if (t256 <= 24 && parts >= 4 && p.K >= ((layout & 2) != 0 ? 3072 : 2048)) return true;
  if ((layout & 2) == 0 && t256 <= 8 && p.K >= 1024) return true;   // (1224 x 136 x 1600 with B k-contiguous: 24 us against 30)
  // (512 x 512 x 2048: 21 us against 25 in half tiles; 192 x 2048 x 2048, 8 tiles: 22.0 against 25.1; 384 x 2048 x 2048, 16:
  // 23.5 against 25.5; at 24 tiles the half tiles are ahead)
  if (layout == 2 && t256 <= 16 && parts >= 4 && p.K >= 2048) return true;
  // (two parts at K = 2048-4095 pay up to a quarter round of tiles -- 192 x 12568 x 3264 with A m-contiguous, 50 tiles: 42 us
  // against 55 whole; 1496 x 80 x 3904: 41 against 63 -- and lose on half a device, 1024 x 8192 x 2048: 56 against 47; with
  // 128 rows or fewer from K = 1024: 8 x 2184 x 1536 with A m-contiguous 24 us against 30, 72 x 2536 x 1408 16 against 19)
  if ((layout & 2) == 0 || p.M <= 128)
    // (few columns likewise: 4968 x 128 x 1856 with B k-contiguous, 20 tiles, 27 us in two parts against 35)
    return p.K >= 4096 || (p.K >= 2048 && (parts >= 4 || t256 <= 96)) ||
           ((p.M <= 128 || p.N <= 128) && p.K >= 1024 && t256 <= 64);
  if (p.K < 4096) return false;
  if (layout == 3) return parts >= 4 || p.K >= 8192;
  // (four parts also while half tiles would fill under 40 % of the device: 1536 x 1536 x 4096, 72 half tiles:
  // 38 us against 46; 512 x 6144 x 4096, 96: 40 against 46)
  const long long th = (long long)((p.M + 127) / 128) * ((p.N + 255) / 256);
  return parts >= 8 || (parts >= 4 && (p.K >= 8192 || p.M <= 192 || th <= 96));
}

// Whether the 128 x 128 quarter tile is the choice: when one round of them holds the problem -- at most a quarter of
// a device's worth of whole tiles -- and the k loop is not so long that cutting it over more units does better.  A
// quarter tile's k loop runs 4.8 us per 1024 k on top of 5 us of launch, first fill and epilogue whatever the tile
// count (one per unit), so its time does not depend on the tile count while that of split-K, shared tiles and half tiles
// does.  Measured against what the other rules picked, all four layouts alike, us:
//   K <= 2048       always: 2048^3 18.5 against 24.3-26.4 (half tiles), 1024 x 2048 x 2048 16.3 against 24.6, 512 x 512 x 1024
//                   10.0 against 15.0, 128 x 512 x 512 (four tiles) 7.3 against 9.7
//   K = 4096        from 48 tiles: 1024 x 4096 x 4096 (256) 31.8 against 42 (shared tiles), 512 x 4096 x 4096 (128) 25.5-26.9
//                   against 38 (split-K), 256 x 4096 x 4096 (64) 25.5 against 28; 256 x 2048 x 4096 (32): 24.4 against 24-26 a tie,
//                   128 x 2048 x 4096 (16): 25 against 18.5 (split-K in sixteen parts)
//   K = 8192        from 112-128 tiles: 512 x 4096 x 8192 (128) 45-46 against 48-52 (split-K), 1024 x 4096 x 8192 (256) 59-60
//                   against 63-66 (shared tiles); 65-96 tiles: 4-11 % behind
//   two rounds (257-512 tiles): 3-20 % behind the half and whole tiles.
// With 64 rows half of every tile is padding: against two k-contiguous operands the streaming kernel stays ahead (64 x 4096 x
// 2048 x . W^T: 11.5 against 14.8), in the other layouts the tile still wins (x . W 14.8 against 16.7 streamed, x^T . W 14.9
// against 21.1 in parts).  With fewer rows a k-contiguous A goes to the streaming kernel or split-K; one that is not has
// neither a streaming kernel nor a 128-row half tile, and the tile wins although it is mostly padding (8 x 14336 x 4096 x^T . W^T
// 25.7 against 31.8 in parts, x^T . W 29.0 against 32.1; 32 x 4096 x 2048 16.8 against 20.9; 16 x 4096 x 1024 17.1 against 20.2).
bool mfma_prefers_quarter(const GemmProblem& p) {
  const int config = mfma_config(p, 14);
  const bool a_kc = (config & 2) != 0, b_kc = (config & 1) != 0;
  if (config == 0 || p.N < 64) return false;
  // (33-63 rows against an n-contiguous weight and a k loop of two or three units: 48 x 4712 x 256 6.6 us against 7.7 in half
  // tiles, 43 x 472 x 256 6.2 against 7.2 streamed; at K = 640 the streaming kernel is ahead again, 24 x 384 x 640 6.3 against 8.1)
  const bool short_nn = a_kc && !b_kc && p.M > 32 && p.K <= 384;
  if (a_kc && !short_nn && (p.M < 64 || (p.M == 64 && b_kc))) return false;
  const long long tq = (long long)((p.M + 127) / 128) * ((p.N + 127) / 128) * p.batch;
  if (tq > compute_units()) return false;
  if (p.batch > 1) {
    // A batch has no split-K pass, so few tiles and a long k loop are no exception (4 x 128 x 128 x 4096: 23.7 us against
    // 40.3 shared; 16 x 128 x 128 x 4096 24.5 against 40.9; 16 x 384 x 384 x 4096, 144 tiles: 45 against 49-56).  But its
    // problems share no operand: with a device's worth of tiles from small problems the operand traffic, twice a half
    // tile's, sets the pace (16 x 512 x 512 x 4096, 256 tiles: 61-75 us against 55-56 shared; 64 x 256 x 256 x 1024: 23.5
    // against 18.7 in half tiles) -- unless a problem alone is 32 tiles or more (4 x 512 x 2048 x 4096: 34.5 against 47).
    // With two or three units per tile the launch is mostly its fixed costs and the traffic does not show (16 x 512 x 512 x 256:
    // 6.5 us against 8.0-8.7 in half tiles; 64 x 256 x 256 x 256: 7.5-7.8 against 8.9-9.9; benchmark config 2, 32 x 256^3 in
    // fp16: 6.4 against 7.0-7.2 in 64 x 64 tiles).
    if (4 * tq <= 3 * compute_units() || tq / p.batch >= 32 || p.K <= 384) return true;
    // (an A that is not k-contiguous has no 128-row half tile to fall back on: 64-row problems, 64 x 64 x 512 x 1024 17-18
    // against 19-23, x 4096: 60 against 70-72; x^T . W with a short k loop, 16 x 256 x 1024 x 1024 18.5 against 23.6)
    return !a_kc && (p.M <= 64 || (!b_kc && p.K <= 1024));
  }
  if (p.K <= 2048) return true;
  // Beyond that the rival is split-K, and what it is worth depends on how deep it can cut (the cut must leave whole stages:
  // 4096 goes in eight parts of 512, but 3200, 4480 or 6016 only in four) and on the partial sums it moves.  Two estimates, in
  // microseconds, fitted to the sweeps:
  //   quarter tiles   5 + 5 per 1024 k, whatever the tile count up to 192, a quarter more at 256
  //   split-K         10 + 20 per 1024 k of a part + the partial sums, parts x M x N x 8 bytes written and read at 7 TB/s;
  //                   on the half tiles that at most 128 rows of a k-contiguous A run on: 9 + 12 per 1024 k + the sums at 5 TB/s
  // measured / estimated for split-K: 256 x 2048 x 4096 in eight 24.2-25.9 / 24.8, 512 x 1536 x 4096 28.4 / 27.2, 512 x 4096 x 8192
  // 48-52 / 49.2, 512 x 3072 x 8192 41.3-42.8 / 44.4, 8 x 1728 x 3200 in four 24.5 / 25.6, 476 x 1936 x 8448 in eight 35.5 / 39.1,
  // 8 x 2848 x 9984 34.1 / 34.6; on half tiles 128 x 2048 x 4096 18.5 / 18.4, 128 x 8192 x 4096 27.5-30 / 28.4; for quarter tiles:
  // K = 3200 20.0 / 20.6, 4096 24.2-25.5 / 25, 4480 26.6 / 26.9, 6016 34.0 / 34.4, 8192 44.7-46.6 / 45, 1024 x 4096 x 8192 (256
  // tiles) 58.7 / 56.3.
  const int parts = mfma_splitk_parts(p);
  if (parts < 2) return true;
  const double part_k = (double)(p.K / parts) / 1024.0;
  const double sums = (double)parts * (double)p.M * (double)p.N * 8.0;   // bytes
  const double split_us = a_kc && p.M <= 128 ? 9.0 + 12.0 * part_k + sums / 5.0e6 : 10.0 + 20.0 * part_k + sums / 7.0e6;
  const double fill = tq > 192 ? 1.0 + 0.25 * (double)(tq - 192) / 64.0 : 1.0;
  const double quarter_us = (5.0 + 5.0 * (double)p.K / 1024.0) * fill;
  return quarter_us <= split_us;
}

// Whether the heuristic takes the tail-sharing form of the 64-deep kernel (tile 10): the tiles left over
// after the whole rounds are cut along k so that every compute unit works on them.  Adding up a tile's
// parts costs about what three quads (768 k) of multiplying do, so it pays for long k loops only.  After
// whole rounds it buys nothing that stands out of the run-to-run spread: a partly filled round runs at
// higher clocks than a full one, and the workgroups leave the shared pieces out of step, which costs the
// whole tiles that follow some of their L2 hits (384 tiles: 151 us against 156; 640 tiles: 241-250 against
// 242-252; 4096 x 11008 x 4096, 176 tiles left over: 270 against 254) -- unless only a handful of tiles
// is left over, which would otherwise cost a round of their own (1536 x 11008 x 4096, 258 tiles: 130 against
// 139 whole and 135 in half tiles).  Otherwise it is taken only where there is no whole round.  Measured against what the other rules pick (us, K = 4096 unless given):
//   64 tiles (three parts)    1024 x 4096 x 4096: 43 against 47-50 (split-K), K = 8192: 64 against 70
//   128 tiles (two parts)     x . W^T: 56-59 against 62-66 (half tiles), K = 8192: 97-100 against 117-122;
//                             x . W: 57-59 against 55-57 (half tiles in one round: those stay), K = 8192: 98-103
//                             against 103-110
//   144 tiles                 3072 x 3072 x 4096: 67-69 against 71-73 (whole tiles)
//   48 tiles                  1536 x 2048 x 4096 x . W^T: 41 against 44 (split-K)
//   below that split-K cuts deeper (32 tiles, K = 16384: 73 against 104); from 160 tiles up whole tiles
//   are as good (160 tiles: 74-76 against 72-75)
bool mfma_prefers_tail(const GemmProblem& p) {
  if (p.K < 2048 || mfma_config(p, 10) == 0) return false;
  const int layout = mfma_layout(p);
  if (narrow_round(p, layout)) return false;   // one round of 256 x 128 half tiles does better
  const long long cus = compute_units();
  const long long t256 = (long long)((p.M + 255) / 256) * ((p.N + 255) / 256) * p.batch;
  const long long th = (long long)((p.M + 127) / 128) * ((p.N + 255) / 256) * p.batch;
  const long long left = t256 % cus;
  // A batch has no split-K pass: under a quarter of a round of tiles this is its only way of cutting k.  From K = 2048
  // when A is not k-contiguous (16 x 256 x 256 x 2048: 29-30 us against 37-39 whole), from 4096 otherwise (4 x 256 x 256 x
  // 4096: 40 us against 44 in half tiles; 48 x 256 x 256 x 8192: 96 against 165), from 8192 for x . W^T of 128 rows or
  // fewer, which the 64 x 64 tiles do well (4 x 128 x 128 x 4096: 39 against 32; 16 x 128 x 128 x 8192: 58 against 72).
  if (p.batch > 1 && t256 < 64) {
    const int from = (layout & 2) == 0 ? 2048 : (layout == 3 && p.M <= 128) ? 8192 : 4096;
    return p.K >= from;
  }
  if (p.K < 4096) {
    // an A that is not k-contiguous (and more than one round of its 256 x 128 half tiles, see above): shared tiles from K =
    // 2048 (1024 x 4096 x 2048, 64 tiles: 32.5 us against 37.7 for split-K; 1536 x 4096 x 2048, 96 tiles: 34.4 against 40.1 whole)
    return (layout & 2) == 0 && t256 >= (p.M >= 512 ? 48 : 64) && t256 <= 128;
  }
  // tiles that are mostly padding rows: 64 x 64 x 512 x 4096, 128 tiles, x . W^T 95 us against 77 for 64 x 64 tiles, with
  // A m-contiguous 92 against 81-82 whole (but 64 x 128 x 128 x 4096 with A m-contiguous: 46 against 70 whole)
  if (p.M <= 64 || (p.M <= 128 && layout == 3)) return false;
  // a last row of tiles that is half padding or more, and half tiles that fit one round (16 x 384 x 384 x 4096: 56 us
  // against 51 in half tiles)
  const int m_rest = p.M % 256;
  if ((layout & 2) != 0 && m_rest >= 1 && m_rest <= 128 && th <= cus) return false;
  if (t256 >= cus) {
    // a handful left over (see above), or one round and up to half of another with a k loop long enough to
    // carry the adding up (3072 x 8192 x 8192, 384 tiles: 275 us against 298)
    // (from K = 4096: 4096 x 6144 x 4096, 384 tiles, 149.8 us against 161.8 whole; 3072 x 8192 x 4096 152.1 against 163.0)
    return left > 0 && (8 * left <= cus || (t256 < 2 * cus && 2 * left <= cus && p.K >= 4096));
  }
  if (left < 48 || left > 160) return false;
  // (the 48-tile figures are of 2-6 rows of tiles, one row stays with split-K; so does K = 8192, which four parts cut
  // deeper: 512 x 6144 x 8192 with A m-contiguous 58 us against 62)
  // (with 1024 rows or more the shared tiles keep K = 8192 too: 1536 x 2048 x 8192 x^T . W^T 64.4 us against 72.5 in parts)
  if (left < 64 && (p.M < 512 || (p.K > 4096 && p.batch == 1 && p.M < 1024))) return false;
  // x . W has half tiles to fall back on: while they fit one round they are as good or better below K = 8192 from 72 tiles
  // up (1536 x 3072 x 4096: 46-53 us in half tiles, 53 shared; 2048 x 3072 x 4096: 48-52 against 51-55)
  // so has x . W^T since its half tiles are 64 deep (whole-line loads): one round of them beats the shared tiles below
  // K = 8192 (1024 x 8192 x 4096: 52.6 us against 57.6; 1536 x 4096 x 4096: 44.9 against 48.5; 2048 x 3072 x 4096: 44.0
  // against 48.7)
  // (from five eighths of a round of them: at half a round the shared tiles are as good or better -- 512 x 8192 x 4096 41.5 us)
  if (layout == 3 && 8 * th >= 5 * cus && th <= cus && p.K < 8192) return false;
  if (left <= (layout == 2 ? 64 : 96)) return true;
  return layout == 3 || (layout & 2) == 0 || p.K >= 8192 || th > cus;
}

hipError_t launch_mfma_splitk(const GemmProblem& p, hipStream_t stream) {
  const int parts = mfma_splitk_parts(p);
  if (parts < 2) return hipErrorInvalidValue;
  const int layout = mfma_layout(p);
  const bool a_kc = (layout & 2) != 0, b_kc = (layout & 1) != 0;
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
  hipError_t e;
  if (a_kc && b_kc && p.M <= 128 && q.K % 64 == 0 && q.K >= 256) {
    // x . W^T: half tiles in their 64-deep form when the parts are whole 64-deep units (128 x 4096 x 4096 20.7 -> 19.8 us,
    // 96 x 11008 x 4096 27.0 -> 26.1; with an n-contiguous B the 32-deep pass is 1-2 % ahead and stays)
    e = p.dtype == srtReal16BF ? launch_m16dh_partial_BF16_11(q, stream) : launch_m16dh_partial_F16_11(q, stream);
  } else if (a_kc && p.M <= 128) {
    if (p.dtype == srtReal16BF) e = b_kc ? launch_m16h_partial_BF16_11(q, stream) : launch_m16h_partial_BF16_10(q, stream);
    else e = b_kc ? launch_m16h_partial_F16_11(q, stream) : launch_m16h_partial_F16_10(q, stream);
  } else if (b_kc && q.K % 64 == 0 && q.K >= 256) {
    // parts that are whole 64-deep units of a k-contiguous B run the 64-deep kernel (1024 x 2048 x 8192 x . W^T: 53.1 ->
    // 49.4 us, x^T . W^T 1-2 %; with an n-contiguous B the two measure the same to +-1 %)
    e = p.dtype == srtReal16BF ? launch_m16d_partial<BF16>(q, a_kc, b_kc, stream)
                               : launch_m16d_partial<F16>(q, a_kc, b_kc, stream);
  } else {
    e = p.dtype == srtReal16BF ? launch_m16_partial<BF16>(q, a_kc, b_kc, stream)
                               : launch_m16_partial<F16>(q, a_kc, b_kc, stream);
  }
  if (e == hipSuccess) {
    const long long lanes = (long long)p.M * (p.N / 8);
    const unsigned blocks = (unsigned)((lanes + 255) / 256);
    if (p.dtype == srtReal16BF)
      hipLaunchKernelGGL(splitk_reduce_kernel<BF16>, dim3(blocks), dim3(256), 0, stream, (const float*)workspace, parts, p);
    else
      hipLaunchKernelGGL(splitk_reduce_kernel<F16>, dim3(blocks), dim3(256), 0, stream, (const float*)workspace, parts, p);
    e = launch_status(stream);
  }
  (void)srtDeviceFree(workspace);   // stream-ordered: reused only by work queued after the kernels above
  return e;
}

const char* mfma_name(int config) {
  switch (config >> 2) {
    case 1: return "mfma_256x256";
    case 4: return "mfma_256x256_k64";
    case 5: return "mfma_256x256_m16";
    case 6: return "mfma_128x256_m16";
    case 9: return "mfma_256x256_m16_k64";
    case 10: return "mfma_256x256_m16_k64_tail";
    case 11: return "mfma_256x256_m16_k64_split";
    case 12: return "mfma_128x256_m16_k64";
    case 13: return "mfma_256x128_m16_k64";
    case 14: return "mfma_128x128_m16_k128";
    case 2: return "mfma_128x128";
    case 7: return "mfma_128x128_any";
    case 8: return "mfma_64x64_any";
    default: return "mfma_64x64";
  }
}

hipError_t launch_mfma(const GemmProblem& p, int config, hipStream_t stream) {
  const int tile = config >> 2;
  const bool a_kc = (config & 2) != 0, b_kc = (config & 1) != 0;
  if (p.dtype == srtReal16BF) return launch_tile<BF16>(p, tile, a_kc, b_kc, stream);
  return launch_tile<F16>(p, tile, a_kc, b_kc, stream);
}

}  // namespace srt
