// 256 x 256 x 64 bf16 / fp16 matmul tile kernel for gfx950 with direct-to-LDS operand staging.
//
// Global memory -> LDS goes through `buffer_load_dwordx4 ... lds`: no staging registers, no
// LDS write instructions, out-of-range addresses return zero (the buffer descriptor bounds
// every operand), and the XOR swizzles below are applied on the *global* side -- lane l of a
// load instruction always lands at LDS byte  M0 + 16 l, so each lane fetches the 16-byte chunk
// that belongs at its landing position.
//
// LDS layouts per operand (one stage = A region 32 KiB + B region 32 KiB, two stages):
//   stored k-contiguous  (A not transposed / B transposed):
//       [256 rows][8 chunks of 16 B]; chunk c of row r sits at position c ^ ((r >> 1) & 7).
//       MFMA operand = one ds_read_b128 (lane l: row l % 32, chunk 2 kk + l / 32).
//   stored mn-contiguous (A transposed / B not transposed):
//       [64 k][32 chunks of 16 B] (a k-row is 256 m or n = 512 B); chunk c of k-row k sits at
//       position c ^ ((k & 3) << 2).  MFMA operand = two ds_read_b64_tr_b16: within each group
//       of 16 lanes the instruction transposes a 4(k) x 16(mn) block, so every lane ends up with
//       4 consecutive k of its own m / n without any VALU work.
//   Both layouts hand lane l the k values kk*16 + 8*(l/32) + 0..7, so any pairing is valid.
//
// Pipeline (per 64-deep k tile t, four phases of 16 MFMAs each):
//   phases 0..2   MFMAs of k slice kk while the LDS reads of slice kk+1 are in flight
//   sync          s_waitcnt vmcnt(0) lgkmcnt(0); s_barrier   -- tile t+1 has landed for every
//                 wave and every wave holds the last slice of tile t in registers
//   phase 3       MFMAs of slice 3, interleaved with the global->LDS loads of tile t+2 (into
//                 the buffer tile t just vacated) and the LDS reads of slice 0 of tile t+1
// One barrier per tile; MFMA issue only pauses for the barrier itself.  The interleave is fixed
// in the source with scheduling fences so each memory instruction issues in an MFMA's shadow.
#pragma once
#include "gemm_common.h"

namespace srt {
namespace dtl {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
#define SRT_LDS __attribute__((address_space(3)))

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int NT = 256;                    // 4 waves, 2 x 2, each 128 x 128
constexpr int REGION = 256 * 128;          // bytes of one operand tile (256 x 64 x 2 B)
constexpr int STAGE = 2 * REGION;
constexpr int LDS_BYTES = 2 * STAGE;       // 128 KiB
constexpr uint32_t OOB = 0x80000000u;      // byte offset beyond any supported operand: reads 0, stores dropped

template <typename T>
__device__ __forceinline__ f32x16_t mfma(u32x4_t a, u32x4_t b, f32x16_t c);
template <>
__device__ __forceinline__ f32x16_t mfma<BF16>(u32x4_t a, u32x4_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b),
                                                 c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x16_t mfma<F16>(u32x4_t a, u32x4_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b),
                                                c, 0, 0, 0);
}

// Raw buffer descriptor: base, stride 0, num_records in bytes, 32-bit untyped data format.
__device__ __forceinline__ u32x4_t make_rsrc(const void* base, uint32_t bytes) {
  const uint64_t p = reinterpret_cast<uint64_t>(base);
  u32x4_t r = {(uint32_t)p, (uint32_t)(p >> 32) & 0xffffu, bytes, 0x00020000u};
  return r;
}

// One 16-byte-per-lane load straight into LDS: lane l's data lands at lds_addr + 16 l.
// Written as inline assembly so that no automatic wait on the vector-memory counter is placed
// in front of unrelated LDS reads; completion is awaited explicitly before the barrier.
__device__ __forceinline__ void load_to_lds(u32x4_t rsrc, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
               : "memory");
}

// ---- global -> LDS ---------------------------------------------------------------------------
// Per-lane byte offsets (into the operand's buffer) of the 8 loads a wave issues per stage for
// one operand; the k advance goes through the scalar offset.
template <bool KC>
struct Loader {
  uint32_t voff[8];
  uint32_t kstep;   // bytes per k tile

  // tile_row0: first m (or n) of the tile.  ld: elements between rows (KC) or between k (MN).
  __device__ __forceinline__ void init(int wave, int lane, int tile_row0, long long ld) {
    if (KC) {
      // load i of this wave covers tile rows (wave*8 + i)*8 .. +7, 8 lanes per row
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int row = (wave * 8 + i) * 8 + (lane >> 3);
        const int chunk = (lane & 7) ^ ((row >> 1) & 7);
        voff[i] = (uint32_t)(((long long)(tile_row0 + row) * ld + chunk * 8) * 2);
      }
      kstep = BK * 2;
    } else {
      // load i covers k rows (wave*8 + i)*2 .. +1, 32 lanes per k row
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int krow = (wave * 8 + i) * 2 + (lane >> 5);
        const int chunk = (lane & 31) ^ ((krow & 3) << 2);
        voff[i] = (uint32_t)(((long long)krow * ld + tile_row0 + chunk * 8) * 2);
      }
      kstep = (uint32_t)(BK * ld * 2);
    }
  }

  // Load i of this wave for the k tile at scalar byte offset `soff` (kt * kstep, or OOB to make
  // the whole load read zeros without touching memory), into the operand region at LDS address
  // `region`.  `tail`: this is a ragged last tile; for a k-contiguous operand the logical chunks
  // >= mask_from lie at or beyond K and must read as zero (an mn-contiguous operand gets that
  // from the bounds check, its k rows >= K being past the end of the view).
  __device__ __forceinline__ void issue_one(u32x4_t rsrc, uint32_t region, int wave, int lane, uint32_t soff, int i,
                                            bool tail, int mask_from) const {
    uint32_t v = voff[i];
    if (KC) {
      // (row >> 1) & 7 of the row this lane fetches depends only on the parity of i
      const int chunk = (lane & 7) ^ ((((i & 1) << 2) + (lane >> 4)) & 7);
      v = (tail && chunk >= mask_from) ? OOB : v;
    }
    load_to_lds(rsrc, region + (uint32_t)(wave * 8 + i) * 1024u, v, soff);
  }
};

// ---- LDS -> MFMA operands ----------------------------------------------------------------------
template <bool KC>
struct FragReader {
  uint32_t base[4];   // KC: one address per kk; MN: one address per 32-wide tile index

  // wave_row0: first m (n) of the wave's 128-wide slice inside the tile
  __device__ __forceinline__ void init(int lane, int wave_row0) {
    if (KC) {
      const int r = lane & 31, h = lane >> 5;
      const int f = (r >> 1) & 7;
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) base[kk] = (uint32_t)((wave_row0 + r) * 128 + (((2 * kk + h) ^ f) << 4));
    } else {
      const int g = lane >> 4, jn = lane & 15, e = jn >> 2, q = jn & 3;
      // lane supplies the address of T[k = 8*(g>>1) + e (+ 16 kk + 4 r)][mn = wave_row0 + 32 t + 16*(g&1) + 4 q]
      const int krow = 8 * (g >> 1) + e;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int mn = wave_row0 + 32 * t + 16 * (g & 1) + 4 * q;
        const int chunk = (mn >> 3) ^ (e << 2);
        base[t] = (uint32_t)(krow * 512 + chunk * 16 + ((mn >> 2) & 1) * 8);
      }
    }
  }

  // operand for 32-wide tile t (0..3) and k slice kk (0..3) of the region at LDS address `region`
  __device__ __forceinline__ u32x4_t read(uint32_t region, int t, int kk) const {
    if (KC) {
      return *reinterpret_cast<const SRT_LDS u32x4_t*>(region + base[kk] + t * 4096);
    } else {
      const uint32_t a = region + base[t] + kk * 8192;
      const u32x2_t lo =
          __builtin_bit_cast(u32x2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<SRT_LDS s16x4_t*>(a)));
      const u32x2_t hi = __builtin_bit_cast(
          u32x2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<SRT_LDS s16x4_t*>(a + 2048)));
      u32x4_t v = {lo.x, lo.y, hi.x, hi.y};
      return v;
    }
  }
};

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

#define SRT_FENCE() __builtin_amdgcn_sched_barrier(0)

template <typename T, bool A_KC, bool B_KC>
__global__ __launch_bounds__(NT) void gemm_dtl_kernel(GemmProblem p) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[];
  const uint32_t lds = (uint32_t)(uintptr_t)(SRT_LDS unsigned char*)lds_raw;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave >> 1) * 128, wn0 = (wave & 1) * 128;

  const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  int tm, tn;
  tile_coords(blockIdx.x, tiles_m, tiles_n, &tm, &tn);
  const int m0 = tm * BM, n0 = tn * BN;
  const int bz = blockIdx.y;

  const uint16_t* A = (const uint16_t*)p.A + (long long)bz * p.sab;
  const uint16_t* B = (const uint16_t*)p.B + (long long)bz * p.sbb;
  const long long lda = A_KC ? p.sam : p.sak;
  const long long ldb = B_KC ? p.sbn : p.sbk;
  // bytes spanned by each operand view: anything beyond reads as zero
  const uint32_t a_bytes = (uint32_t)((A_KC ? (long long)(p.M - 1) * lda + p.K : (long long)(p.K - 1) * lda + p.M) * 2);
  const uint32_t b_bytes = (uint32_t)((B_KC ? (long long)(p.N - 1) * ldb + p.K : (long long)(p.K - 1) * ldb + p.N) * 2);
  const u32x4_t ra = make_rsrc(A, a_bytes);
  const u32x4_t rb = make_rsrc(B, b_bytes);

  Loader<A_KC> la;
  Loader<B_KC> lb;
  la.init(wave, lane, m0, lda);
  lb.init(wave, lane, n0, ldb);
  FragReader<A_KC> fa;
  FragReader<B_KC> fb;
  fa.init(lane, wm0);
  fb.init(lane, wn0);

  f32x16_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  const int KT = (p.K + BK - 1) / BK;
  // first logical 16-byte chunk of the last k tile that lies at or beyond K (8 = tile is whole)
  const int tail_mask = (p.K % BK) ? ((p.K % BK) + 7) / 8 : 8;

  // ---- prologue: tiles 0 and 1 in flight, wait for tile 0 only ----
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const uint32_t stage = lds + (uint32_t)t * STAGE;
    const bool tail = (t == KT - 1) && tail_mask < 8;
    const uint32_t soa = t < KT ? (uint32_t)t * la.kstep : OOB;
    const uint32_t sob = t < KT ? (uint32_t)t * lb.kstep : OOB;
#pragma unroll
    for (int i = 0; i < 8; ++i) la.issue_one(ra, stage, wave, lane, soa, i, tail, tail_mask);
#pragma unroll
    for (int i = 0; i < 8; ++i) lb.issue_one(rb, stage + REGION, wave, lane, sob, i, tail, tail_mask);
  }
  asm volatile("s_waitcnt vmcnt(16)\n\ts_barrier" ::: "memory");
  SRT_FENCE();

  u32x4_t af[2][4], bf[2][4];   // [register set][32-wide tile]
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    af[0][t] = fa.read(lds, t, 0);
    bf[0][t] = fb.read(lds + REGION, t, 0);
  }

  // The loop body is branch-free: loads past the last tile are aimed out of range (they return
  // zeros without touching memory and land in a buffer nobody reads again), and the reads of
  // "tile KT" in the last trip fetch LDS contents that are never used.
  for (int kt = 0; kt < KT; ++kt) {
    const uint32_t cur = lds + (uint32_t)(kt & 1) * STAGE;
    const uint32_t nxt = lds + (uint32_t)((kt + 1) & 1) * STAGE;

    // ---- phases 0..2: MFMAs of slice kk, reads of slice kk+1 ----
#pragma unroll
    for (int kk = 0; kk < 3; ++kk) {
      const int s = kk & 1;   // register set holding slice kk
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] = mfma<T>(af[s][i], bf[s][j], acc[i][j]);
          // one operand fragment of the next slice every second MFMA
          if ((j & 1) == 0) {
            const int u = i * 2 + (j >> 1);   // 0..7
            if (u < 4) af[s ^ 1][u] = fa.read(cur, u, kk + 1);
            else bf[s ^ 1][u - 4] = fb.read(cur + REGION, u - 4, kk + 1);
          }
          SRT_FENCE();
        }
      }
    }

    // ---- sync: slice 3 of this tile is in registers, tile kt+1 has landed ----
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    SRT_FENCE();

    // ---- phase 3: MFMAs of slice 3 (register set 1), loads of tile kt+2 into the buffer just
    //      vacated, reads of slice 0 of tile kt+1 ----
    const int k2 = kt + 2;
    const bool tail = (k2 == KT - 1) && tail_mask < 8;
    const uint32_t soa = k2 < KT ? (uint32_t)k2 * la.kstep : OOB;
    const uint32_t sob = k2 < KT ? (uint32_t)k2 * lb.kstep : OOB;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[i][j] = mfma<T>(af[1][i], bf[1][j], acc[i][j]);
        const int g = i * 4 + j;   // 0..15: one global->LDS load per MFMA
        if (g < 8) la.issue_one(ra, cur, wave, lane, soa, g, tail, tail_mask);
        else lb.issue_one(rb, cur + REGION, wave, lane, sob, g - 8, tail, tail_mask);
        if ((j & 1) == 0) {
          const int u = i * 2 + (j >> 1);
          if (u < 4) af[0][u] = fa.read(nxt, u, 0);
          else bf[0][u - 4] = fb.read(nxt + REGION, u - 4, 0);
        }
        SRT_FENCE();
      }
    }
  }
  // the loads issued in the last trip (all out of range) must retire before the LDS is released
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");

  // ---- epilogue: bias + activation on the fp32 accumulators, one rounding, 16-bit stores ----
  // lane holds column l % 32 and rows 8*(v/4) + 4*(l/32) + v%4 of each 32 x 32 tile.  Stores go
  // through a bounds-checked buffer; lanes outside M x N aim at an out-of-range offset.
  Epilogue<T> ep(p);
  uint16_t* C = (uint16_t*)p.C + (long long)bz * p.scb;
  const long long c_last = (long long)(p.M - 1) * p.scm + p.N;   // elements spanned by C (< 2^30, checked on the host)
  const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc(C, 0, (int)(c_last * 2), 0x00020000);
  const int ldc2 = (int)(p.scm * 2);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + wn0 + 32 * j + (lane & 31);
    const bool n_ok = n < p.N;
    const float bcol = (ep.per_row || !n_ok) ? 0.0f : ep.bias_at(0, n);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm0 + 32 * i + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        const bool ok = n_ok && m < p.M;
        const float bv = ep.per_row ? (ok ? ep.bias_at(m, n) : 0.0f) : bcol;
        const uint32_t off = ok ? (uint32_t)(m * ldc2 + n * 2) : OOB;
        __builtin_amdgcn_raw_buffer_store_b16((short)ep.finish(acc[i][j][v], bv), rc, (int)off, 0, 0);
      }
    }
  }
}

#undef SRT_FENCE

// Host-side preconditions beyond those of the MFMA family: every operand view must span less
// than 2 GiB so 32-bit buffer offsets reach it, including the rows of the last (partial) tile.
inline bool dtl_fits(const GemmProblem& p, bool a_kc, bool b_kc) {
  const long long lda = a_kc ? p.sam : p.sak, ldb = b_kc ? p.sbn : p.sbk;
  const long long a_reach = a_kc ? ((long long)p.M + BM) * lda + p.K : ((long long)p.K + BK) * lda + p.M + BM;
  const long long b_reach = b_kc ? ((long long)p.N + BN) * ldb + p.K : ((long long)p.K + BK) * ldb + p.N + BN;
  const long long c_reach = ((long long)p.M + BM) * p.scm + p.N + BN;
  const long long lim = 0x7fffffffLL / 2 - 4096;   // in elements: byte offsets stay below 2^31
  return a_reach < lim && b_reach < lim && c_reach < lim;
}

template <typename T, bool A_KC, bool B_KC>
hipError_t launch(const GemmProblem& p, hipStream_t stream) {
  auto kernel = gemm_dtl_kernel<T, A_KC, B_KC>;
  static bool configured = false;   // benign race: setting the attribute twice is harmless
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
    if (e != hipSuccess) return e;
    configured = true;
  }
  const int tiles = ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
  hipLaunchKernelGGL(kernel, dim3(tiles, p.batch), dim3(NT), LDS_BYTES, stream, p);
  return hipGetLastError();
}

}  // namespace dtl
}  // namespace srt
