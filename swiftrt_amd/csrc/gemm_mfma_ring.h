// 256 x 256 bf16 / fp16 matmul tile kernel for gfx950: direct-to-LDS operand staging through a
// ring of NS k-stages of depth 32, v_mfma_f32_32x32x16 with fp32 accumulators in registers,
// fused bias + activation epilogue staged through LDS into 16-byte row stores.
//
// Why a ring of shallow stages: a global load takes on the order of a microsecond to land, i.e.
// longer than the 64 MFMAs of a 64-deep k tile take to issue.  What bounds the prefetch distance
// is LDS capacity, so the 160 KiB are cut into NS = 5 stages of 32 KiB (k depth 32): a stage is
// requested (NS - 1) iterations -- about 4 x 1024 MFMA cycles -- before it is consumed.
//
// Global memory -> LDS goes through `buffer_load_dwordx4 ... lds`: no staging registers, no LDS
// write instructions, out-of-range addresses return zero (the buffer descriptor bounds every
// operand), and the XOR swizzles are applied on the *global* side -- lane l of a load always
// lands at LDS byte M0 + 16 l, so each lane fetches the 16-byte chunk that belongs at its
// landing position.
//
// LDS layouts per operand (one stage = A region 16 KiB + B region 16 KiB):
//   stored k-contiguous  (A not transposed / B transposed):
//       [256 rows][4 chunks of 16 B]; chunk c of row r sits at position c ^ ((r >> 2) & 3).
//       MFMA operand = one ds_read_b128 (lane l: row l % 32, chunk 2 kk + l / 32).
//   stored mn-contiguous (A transposed / B not transposed):
//       [32 k][32 chunks of 16 B] (a k-row is 256 m or n = 512 B); chunk c of k-row k sits at
//       position c ^ ((k & 3) << 2).  MFMA operand = two ds_read_b64_tr_b16: within each group
//       of 16 lanes the instruction transposes a 4(k) x 16(mn) block, so every lane ends up with
//       4 consecutive k of its own m / n without any VALU work.
//   Both layouts hand lane l the k values kk*16 + 8*(l/32) + 0..7, so any pairing is valid, and
//   both are free of LDS bank conflicts (measured: SQ_LDS_BANK_CONFLICT = 0).
//
// Pipeline, per stage s (two phases of 16 MFMAs per wave):
//   phase 0   MFMAs of k slice 0 (registers); the LDS reads of slice 1 ride on the first eight
//             MFMAs, the four B loads of stage s-1+NS on the last eight
//   sync      s_waitcnt vmcnt(8 (NS-2)) lgkmcnt(0); s_barrier -- stage s+1 has landed for every
//             wave, and every wave holds all of stage s in registers, so slot s % NS is free
//   phase 1   MFMAs of slice 1, interleaved with the four A loads of stage s+NS (into the slot
//             just freed) and the LDS reads of slice 0 of stage s+1
// The interleave is fixed in the source with scheduling fences so that every memory instruction
// issues in the shadow of an MFMA.
//
// The MFMA is issued with the B fragment as its first operand, so each 32 x 32 accumulator tile
// is C^T: a lane owns one row m and, per group of four registers, four consecutive columns n --
// the epilogue rounds them, packs 8 bytes per group into an LDS staging area and writes C from
// there in whole 256-byte row segments.
#pragma once
#include "gemm_common.h"

#include <type_traits>

namespace srt {
namespace ring {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
#define SRT_LDS __attribute__((address_space(3)))
// Cache policy of the result stores: non-temporal.  C is written once and never re-read by the
// kernel, so its lines should not displace operand lines in L2 nor wait there for the
// end-of-kernel write-back (measured: -9 us per 8192^3 launch).
#ifndef SRT_STORE_AUX
#define SRT_STORE_AUX 2   // bit 1 of the buffer instruction's cache-policy field = nt
#endif

constexpr int BM = 256, BN = 256, BK = 32;
constexpr int NT = 256;                    // 4 waves, 2 x 2, each 128 x 128
constexpr int REGION = 256 * BK * 2;       // bytes of one operand stage (16 KiB)
constexpr int STAGE = 2 * REGION;          // 32 KiB
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

// The same load in two halves, for the main loop: the LDS landing address goes into M0 first,
// an MFMA is issued in between (it also provides the wait state M0 needs before the load reads
// it), then the load itself.  Nothing else may touch M0 between the two.
template <int IMM>
__device__ __forceinline__ void set_lds_target(uint32_t lds_base) {
  asm volatile("s_add_u32 m0, %0, %1" : : "s"(lds_base), "n"(IMM) : "scc");
}
__device__ __forceinline__ void load_to_lds_at_m0(u32x4_t rsrc, uint32_t voff, uint32_t soff) {
  asm volatile("buffer_load_dwordx4 %0, %1, %2 offen lds" : : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}

// ---- global -> LDS ---------------------------------------------------------------------------
// Per-lane byte offsets (into the operand's buffer) of the 4 loads a wave issues per stage for
// one operand; the tile's position and the k advance go through the scalar offset.
template <bool KC>
struct Loader {
  uint32_t voff[4];

  // tile_row0: first m (or n) of the tile.  ld: elements between rows (KC) or between k (MN).
  __device__ __forceinline__ void init(int wave, int lane, int tile_row0, long long ld) {
    if (KC) {
      // load i of this wave covers tile rows (wave*4 + i)*16 .. +15, 4 lanes per 64-byte row
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int row = (wave * 4 + i) * 16 + (lane >> 2);
        const int chunk = (lane & 3) ^ ((row >> 2) & 3);
        voff[i] = (uint32_t)(((long long)(tile_row0 + row) * ld + chunk * 8) * 2);
      }
    } else {
      // load i covers k rows (wave*4 + i)*2 .. +1, 32 lanes per 512-byte k row
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int krow = (wave * 4 + i) * 2 + (lane >> 5);
        const int chunk = (lane & 31) ^ ((krow & 3) << 2);
        voff[i] = (uint32_t)(((long long)krow * ld + tile_row0 + chunk * 8) * 2);
      }
    }
  }

  // Load i of this wave for the k stage at scalar byte offset `soff` (tile offset + stage * kstep,
  // or OOB to make the whole load read zeros without touching memory), into the operand region
  // at LDS address `region`.  `tail`: this is a ragged last stage holding only `krem` (< BK) k
  // values; what lies at or beyond K must read as zero: for a k-contiguous operand the logical
  // 16-byte chunks >= ceil(krem / 8) of every row, for an mn-contiguous one the k rows >= krem.
  __device__ __forceinline__ void issue_one(u32x4_t rsrc, uint32_t region, int wave, int lane, uint32_t soff, int i,
                                            bool tail, int krem) const {
    uint32_t v = voff[i];
    if (tail && beyond_k(wave, lane, i, krem)) v = OOB;
    load_to_lds(rsrc, region + (uint32_t)(wave * 4 + i) * 1024u, v, soff);
  }

  // does load i of this lane fetch k values at or beyond K in a ragged last stage of krem values?
  __device__ __forceinline__ bool beyond_k(int wave, int lane, int i, int krem) const {
    if (KC) {
      // (row >> 2) & 3 of the row this lane fetches does not depend on i or the wave
      const int chunk = (lane & 3) ^ ((lane >> 4) & 3);
      return chunk >= (krem + 7) / 8;
    }
    return (wave * 4 + i) * 2 + (lane >> 5) >= krem;
  }

  // Aim what lies at or beyond K out of range for good (called just before the loads of a ragged
  // last stage are issued; the per-lane state is derived afresh for the next tile).
  __device__ __forceinline__ void mask_tail(int wave, int lane, int krem) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (beyond_k(wave, lane, i, krem)) voff[i] = OOB;
  }
};

// ---- LDS -> MFMA operands ----------------------------------------------------------------------
template <bool KC>
struct FragReader {
  uint32_t base[4];   // KC: [0..1] one address per k slice; MN: one address per 32-wide tile index

  // wave_row0: first m (n) of the wave's 128-wide slice inside the tile
  __device__ __forceinline__ void init(int lane, int wave_row0) {
    if (KC) {
      const int r = lane & 31, h = lane >> 5;
      const int f = (r >> 2) & 3;
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) base[kk] = (uint32_t)((wave_row0 + r) * 64 + (((2 * kk + h) ^ f) << 4));
      base[2] = base[3] = 0;
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

  // operand for 32-wide tile t (0..3) and k slice kk (0..1) of the region at LDS address `region`
  __device__ __forceinline__ u32x4_t read(uint32_t region, int t, int kk) const {
    if (KC) {
      return *reinterpret_cast<const SRT_LDS u32x4_t*>(region + base[kk] + t * 2048);
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
// An empty statement that "rewrites" an accumulator tile in the accumulator registers.  After an
// MFMA it ties the MFMA to its place in the instruction stream (MFMAs have no side effects;
// without this the compiler is free to gather them elsewhere).  In the epilogue it ends the life
// of the copies the compiler makes in ordinary registers to test or convert accumulators, which
// it would otherwise keep -- and spill -- until their next use.
__device__ __forceinline__ void pin(f32x16_t& acc) { asm volatile("" : "+a"(acc)); }
__device__ __forceinline__ void pin_all(f32x16_t (&acc)[4][4]) {
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) pin(acc[i][j]);
}

// Epilogue of one wave.
// acc[i][j] is a transposed 32 x 32 tile: lane l owns row m = wave_m0 + 32 i + l % 32 and, in
// registers 4 g .. 4 g + 3, the columns n = wave_n0 + 32 j + 8 g + 4 (l / 32) + 0..3.
//
// Step 1 for identity / relu / clippedRelu (load_bias): the bias values a lane adds -- 64
// per-column ones, or 4 per-row ones after a C^T flip -- are requested in one batch right after
// the k loop, ahead of the wait and barrier that end it, so their latency passes while the matrix
// pipe drains (read where they are used they came in sixteen dependent rounds of a global load's
// latency each).  They wait in their stored 16-bit form, two to a register: b[4 j + g] holds the
// four values of column group (j, g); in the per-row case b[i].x holds row tile i's value.  A
// dense, 8-byte-aligned bias is read as sixteen 8-byte loads.  Bias, then the activation as one or
// two min/max instructions, are applied in store_tile to the copy that leaves the accumulator
// registers, in straight-line code; HAS_BIAS and CLAMP are compile-time so each variant carries
// only the instructions it needs (with HAS_BIAS a null bias pointer adds nothing).  CLAMP: 0 none,
// 1 relu = max(x, 0), 2 clippedRelu = min(max(x, 0), coef).  max(NaN, 0) is 0 on this hardware,
// which is also what x > 0 ? x : 0 gives.
template <typename T>
__device__ __forceinline__ void load_bias(const GemmProblem& p, int wave_m0, int wave_n0, int lane, u32x2_t (&b)[16]) {
  using S = typename T::storage;
  static_assert(sizeof(S) == 2, "16-bit element types");
  const S* bias = (const S*)p.bias;
  const int r = lane & 31, h = lane >> 5;
#pragma unroll
  for (int c = 0; c < 16; ++c) b[c] = u32x2_t{0u, 0u};
  if (!bias) return;
  if (p.bias_per_row) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = wave_m0 + 32 * i + r;
      if (m < p.M) b[i].x = bias[(long long)m * p.sbias];
    }
  } else if (p.sbias == 1 && (reinterpret_cast<uintptr_t>(bias) & 7u) == 0) {
    // N is a multiple of 8 and n of 4: a lane's four columns are all inside or all outside
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      const int n = wave_n0 + 8 * c + 4 * h;
      if (n < p.N) b[c] = *reinterpret_cast<const u32x2_t*>(bias + n);
    }
  } else {
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      uint32_t v[4] = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int n = wave_n0 + 8 * c + 4 * h + e;
        if (n < p.N) v[e] = bias[(long long)n * p.sbias];
      }
      b[c] = u32x2_t{v[0] | (v[1] << 16), v[2] | (v[3] << 16)};
    }
  }
}

// Step 2 (store_tile): one rounding to the element type, then a trip through LDS so that global
// stores are whole 16-byte chunks of C rows (a store instruction writes four 256-byte row
// segments instead of 64 scattered pieces).  The wave's 128 x 128 result goes in two halves of
// 64 rows through its private 16 KiB staging area at LDS address `stage`: [64 rows][16 chunks of
// 16 B], chunk c of row r at position c ^ (r & 15) (reads of a row are conflict-free, writes of
// a column 2-way).  Global stores go through a bounds-checked buffer; chunks outside M x N aim
// out of range.
// Rounding uses the one-instruction hardware converter, which rounds to nearest even like the
// reference's encoder but leaves a NaN some quiet-NaN pattern where the reference stores 0x7FFF:
// the values are tested as they are converted, and for a half in which any lane of the wave saw
// a NaN every NaN pattern is rewritten to 0x7FFF on its way from the staging area to memory.
__device__ __forceinline__ uint32_t canonical_nans_bf16x2(uint32_t w) {
  const uint32_t lo = w & 0xffffu, hi = w >> 16;
  const uint32_t l = (lo & 0x7fffu) > 0x7f80u ? 0x7fffu : lo;
  const uint32_t u = (hi & 0x7fffu) > 0x7f80u ? 0x7fffu : hi;
  return l | (u << 16);
}
template <typename T, bool HAS_BIAS, int CLAMP>
__device__ __forceinline__ void store_tile(const GemmProblem& p, const f32x16_t (&acc)[4][4], int wave_m0, int wave_n0,
                                           int bz, int lane, uint32_t stage, const u32x2_t (&b)[16]) {
  using S = typename T::storage;
  const bool per_row = p.bias_per_row != 0;
  const float ceiling = p.coef;
  constexpr bool FIXUP = T::dtype == srtReal16BF;   // the fp16 converter already encodes NaNs as required
  S* C = (S*)p.C + (long long)bz * p.scb;
  const long long c_last = (long long)(p.M - 1) * p.scm + p.N;   // elements spanned by C (< 2^30, checked on the host)
  const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc(C, 0, (int)(c_last * 2), 0x00020000);
  const int ldc2 = (int)(p.scm * 2);
  const int r = lane & 31, h = lane >> 5;
  // read side: lane covers chunk (lane & 15) of rows (lane >> 4) + 4 it
  const int rd_chunk = lane & 15, rd_row = lane >> 4;
  const int n_rd = wave_n0 + 8 * rd_chunk;
  const bool n_rd_ok = n_rd < p.N;   // N is a multiple of 8 (checked on the host): the chunk is whole

#pragma unroll
  for (int half = 0; half < 2; ++half) {
    // ---- registers -> staging (fenced per accumulator tile so that the compiler does not pull
    //      all the accumulator reads of a half, or of the next half, to the front) ----
    bool nan = false;
#pragma unroll
    for (int ii = 0; ii < 2; ++ii) {
      const int i = 2 * half + ii;
      const int row = 32 * ii + r;
      const uint32_t row_addr = stage + (uint32_t)row * 256u + (uint32_t)h * 8u;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        SRT_FENCE();
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          float a0 = acc[i][j][4 * g], a1 = acc[i][j][4 * g + 1], a2 = acc[i][j][4 * g + 2], a3 = acc[i][j][4 * g + 3];
          // one copy out of the accumulator registers, here, for both the test and the conversion
          asm volatile("" : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3));
          const int c = 4 * j + g;
          if (HAS_BIAS) {
            const float br = T::to_float((S)(b[i].x & 0xffffu));
            a0 += per_row ? br : T::to_float((S)(b[c].x & 0xffffu));
            a1 += per_row ? br : T::to_float((S)(b[c].x >> 16));
            a2 += per_row ? br : T::to_float((S)(b[c].y & 0xffffu));
            a3 += per_row ? br : T::to_float((S)(b[c].y >> 16));
          }
          if (CLAMP >= 1) {
            a0 = __builtin_fmaxf(a0, 0.0f); a1 = __builtin_fmaxf(a1, 0.0f);
            a2 = __builtin_fmaxf(a2, 0.0f); a3 = __builtin_fmaxf(a3, 0.0f);
          }
          if (CLAMP == 2) {
            a0 = __builtin_fminf(a0, ceiling); a1 = __builtin_fminf(a1, ceiling);
            a2 = __builtin_fminf(a2, ceiling); a3 = __builtin_fminf(a3, ceiling);
          }
          if (FIXUP) nan |= __builtin_isunordered(a0, a1) | __builtin_isunordered(a2, a3);
          const u32x2_t w = {T::template pack2<false>(a0, a1), T::template pack2<false>(a2, a3)};
          *reinterpret_cast<SRT_LDS u32x2_t*>(row_addr + (uint32_t)((c ^ (row & 15)) << 4)) = w;
        }
      }
    }
    SRT_FENCE();
    const bool fix = FIXUP && __builtin_amdgcn_ballot_w64(nan) != 0;
    // ---- staging -> global: 16 instructions of 4 rows x 256 bytes, read four at a time ----
#pragma unroll
    for (int it4 = 0; it4 < 4; ++it4) {
      u32x4_t v[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int row = rd_row + 4 * (4 * it4 + q);
        v[q] = *reinterpret_cast<const SRT_LDS u32x4_t*>(stage + (uint32_t)row * 256u + (uint32_t)((rd_chunk ^ (row & 15)) << 4));
      }
      if (fix) {   // rare: some accumulator of this half was a NaN
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int e = 0; e < 4; ++e) v[q][e] = canonical_nans_bf16x2(v[q][e]);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int row = rd_row + 4 * (4 * it4 + q);
        const int m = wave_m0 + 64 * half + row;
        const uint32_t off = (n_rd_ok && m < p.M) ? (uint32_t)(m * ldc2 + n_rd * 2) : OOB;
        __builtin_amdgcn_raw_buffer_store_b128(v[q], rc, (int)off, 0, SRT_STORE_AUX);
      }
      SRT_FENCE();
    }
  }
}

// Epilogue for sigmoid / tanh / elu: acc + bias goes to the staging area as fp32, and the
// activation, the rounding and the store run in a rolled loop over the staged rows, so the
// transcendental code exists once instead of once per accumulator register.
// Four passes of 32 rows: staging is [32 rows][32 chunks of 16 B], chunk c of row r at c ^ r.
template <typename T>
__device__ __forceinline__ void store_tile_transcendental(const GemmProblem& p, const f32x16_t (&acc)[4][4],
                                                          int wave_m0, int wave_n0, int bz, int lane, uint32_t stage,
                                                          const u32x2_t (&b)[16]) {
  using S = typename T::storage;
  S* C = (S*)p.C + (long long)bz * p.scb;
  const long long c_last = (long long)(p.M - 1) * p.scm + p.N;
  const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc(C, 0, (int)(c_last * 2), 0x00020000);
  const int ldc2 = (int)(p.scm * 2);
  const bool per_row = p.bias_per_row != 0;
  const int r = lane & 31, h = lane >> 5;
  const int rd_chunk = lane & 31, rd_row = lane >> 5;   // read side: 4 columns of rows rd_row + 2 it
  const int n_rd = wave_n0 + 4 * rd_chunk;
  const bool n_rd_ok = n_rd < p.N;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    // bias from the registers load_bias filled before the tile's first store was issued: a global load in
    // here would wait, with its vmcnt(0), for every store of the previous pass as well
    const float brow = T::to_float((S)(b[i].x & 0xffffu));
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const u32x2_t bw = b[4 * j + g];
        const float bcol[4] = {T::to_float((S)(bw.x & 0xffffu)), T::to_float((S)(bw.x >> 16)),
                               T::to_float((S)(bw.y & 0xffffu)), T::to_float((S)(bw.y >> 16))};
        f32x4_t x;
#pragma unroll
        for (int e = 0; e < 4; ++e) x[e] = acc[i][j][4 * g + e] + (per_row ? brow : bcol[e]);
        const int c = 8 * j + 2 * g + h;
        *reinterpret_cast<SRT_LDS f32x4_t*>(stage + (uint32_t)r * 512u + (uint32_t)((c ^ r) << 4)) = x;
      }
    // the staged values' activation, rounding and store: one copy of the loop per activation, chosen by a
    // uniform branch (a switch per element inside the loop costs a chain of branches each)
    auto tail = [&](auto act) __attribute__((always_inline)) {
      constexpr int ACT = decltype(act)::value;
#pragma unroll 4
      for (int it = 0; it < 16; ++it) {
        const int row = rd_row + 2 * it;
        const f32x4_t x =
            *reinterpret_cast<const SRT_LDS f32x4_t*>(stage + (uint32_t)row * 512u + (uint32_t)((rd_chunk ^ row) << 4));
        uint32_t lo = (uint32_t)T::from_float(activation16_ct<ACT>(p.coef, x[0])) |
                      ((uint32_t)T::from_float(activation16_ct<ACT>(p.coef, x[1])) << 16);
        uint32_t hi = (uint32_t)T::from_float(activation16_ct<ACT>(p.coef, x[2])) |
                      ((uint32_t)T::from_float(activation16_ct<ACT>(p.coef, x[3])) << 16);
        const u32x2_t w = {lo, hi};
        const int mm = wave_m0 + 32 * i + row;
        const uint32_t off = (n_rd_ok && mm < p.M) ? (uint32_t)(mm * ldc2 + n_rd * 2) : OOB;
        __builtin_amdgcn_raw_buffer_store_b64(w, rc, (int)off, 0, SRT_STORE_AUX);
      }
    };
    if (p.activation == srtActivationSigmoid) tail(std::integral_constant<int, srtActivationSigmoid>{});
    else if (p.activation == srtActivationTanh) tail(std::integral_constant<int, srtActivationTanh>{});
    else tail(std::integral_constant<int, srtActivationElu>{});
  }
}

// EPI selects the epilogue the kernel is compiled with (the accumulators never cross a branch).
constexpr int EPI_PLAIN = 0;       // matmul: no bias, identity
constexpr int EPI_BIAS = 1;        // bias, identity
constexpr int EPI_RELU = 2;        // relu
constexpr int EPI_BIAS_RELU = 3;   // bias, relu (the Dense configuration)
constexpr int EPI_CLIPPED = 4;     // clippedRelu, bias optional (a null bias adds nothing)
constexpr int EPI_TRANS = 5;       // sigmoid / tanh / elu (+ bias)

template <typename T, int EPI>
__device__ __forceinline__ void store_tile_linear(const GemmProblem& p, const f32x16_t (&acc)[4][4], int wave_m0,
                                                  int wave_n0, int bz, int lane, uint32_t stage, const u32x2_t (&b)[16]) {
  if (EPI == EPI_BIAS) store_tile<T, true, 0>(p, acc, wave_m0, wave_n0, bz, lane, stage, b);
  else if (EPI == EPI_RELU) store_tile<T, false, 1>(p, acc, wave_m0, wave_n0, bz, lane, stage, b);
  else if (EPI == EPI_BIAS_RELU) store_tile<T, true, 1>(p, acc, wave_m0, wave_n0, bz, lane, stage, b);
  else if (EPI == EPI_CLIPPED) store_tile<T, true, 2>(p, acc, wave_m0, wave_n0, bz, lane, stage, b);   // a null bias adds nothing
  else store_tile<T, false, 0>(p, acc, wave_m0, wave_n0, bz, lane, stage, b);
}


// One tile as the loads see it: the byte offsets of its first row (column) inside the operand
// tensors, batch offset included.  All scalar.
struct TileRef {
  uint32_t offa, offb;
  int m0, n0, bz;
};

template <bool A_KC, bool B_KC>
__device__ __forceinline__ TileRef locate_tile(const GemmProblem& p, int v, int tiles_m, int tiles_n) {
  const int per_batch = tiles_m * tiles_n;
  const int bz = v / per_batch;
  int tm, tn;
  tile_coords(v - bz * per_batch, tiles_m, tiles_n, &tm, &tn);
  TileRef t;
  t.m0 = tm * BM;
  t.n0 = tn * BN;
  t.bz = bz;
  const long long lda = A_KC ? p.sam : p.sak;
  const long long ldb = B_KC ? p.sbn : p.sbk;
  t.offa = (uint32_t)(((long long)bz * p.sab + (A_KC ? (long long)t.m0 * lda : (long long)t.m0)) * 2);
  t.offb = (uint32_t)(((long long)bz * p.sbb + (B_KC ? (long long)t.n0 * ldb : (long long)t.n0)) * 2);
  return t;
}

// The kernel is persistent: the grid has one workgroup per compute unit (or per tile when there
// are fewer tiles), and workgroup w computes tiles w, w + G, w + 2 G, ... of the XCD-aware order.
// The k loop runs across tile boundaries: while the last stages of a tile are multiplied, the
// ring slots they vacate receive the first NS - 2 stages of the workgroup's next tile, so that
// tile starts with its operands already in LDS; the two slots vacated last are the epilogue's
// staging area, and the remaining stages of the next tile's ring are requested right after the
// epilogue.  With a ragged last k stage or fewer than NS stages the overlap is off and the next
// tile starts from a full prologue.
template <typename T, bool A_KC, bool B_KC, int EPI, int NS>
__global__ __launch_bounds__(NT) void gemm_ring_kernel(GemmProblem p) {
  static_assert(NS == 5, "ring depth");   // slot arithmetic below assumes the staging slots are NS-2, NS-1 ahead
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[];
  const uint32_t lds = (uint32_t)(uintptr_t)(SRT_LDS unsigned char*)lds_raw;

  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  // The lane id is worked out afresh (two instructions) wherever per-lane state is derived from
  // it, instead of being held in a register for the life of the kernel.
  auto lane_id = []() {
    uint32_t zero = 0;
    asm volatile("" : "+s"(zero));   // opaque: keeps the two instructions where they are written
    return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, zero));
  };
  const int wm0 = (wave >> 1) * 128, wn0 = (wave & 1) * 128;

  const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  const int total = tiles_m * tiles_n * p.batch;
  const int grid = (int)gridDim.x;
  int v = (int)blockIdx.x;

  const long long lda = A_KC ? p.sam : p.sak;
  const long long ldb = B_KC ? p.sbn : p.sbk;
  // One descriptor per operand, spanning the views of all batches: anything beyond the last
  // batch's view reads as zero.  Inside the tensor nothing is masked by the descriptor: rows of a
  // partial tile beyond M (columns beyond N) read whatever follows and only reach accumulators
  // that are never stored; k beyond K is masked by the loaders (ragged last stage).
  const long long a_view = A_KC ? (long long)(p.M - 1) * lda + p.K : (long long)(p.K - 1) * lda + p.M;
  const long long b_view = B_KC ? (long long)(p.N - 1) * ldb + p.K : (long long)(p.K - 1) * ldb + p.N;
  const u32x4_t ra = make_rsrc(p.A, (uint32_t)(((long long)(p.batch - 1) * p.sab + a_view) * 2));
  const u32x4_t rb = make_rsrc(p.B, (uint32_t)(((long long)(p.batch - 1) * p.sbb + b_view) * 2));
  const uint32_t kstep_a = A_KC ? (uint32_t)(BK * 2) : (uint32_t)(BK * lda * 2);   // bytes per k stage
  const uint32_t kstep_b = B_KC ? (uint32_t)(BK * 2) : (uint32_t)(BK * ldb * 2);
  const int KT = (p.K + BK - 1) / BK;
  const int krem = p.K % BK;   // k values in a ragged last stage (0: the stage is whole)
  const bool ragged = krem != 0;
  const bool overlap = !ragged && KT >= NS;

  // With A stored k x m (transposed lhs) the k stages are walked in rotated order, starting at a
  // stage that depends on the XCD the workgroup runs on (its id mod 8): k rows of A are a power
  // of two apart, so every workgroup reading the same k hits the same few memory channels, and
  // spreading the eight XCDs over k measured +4 %.  The workgroups of one XCD keep a common
  // start: they share operand panels through their L2 only while they read the same k range at
  // about the same time.  For k-contiguous A the common start of all XCDs is kept: there the
  // last-level cache reuse between XCDs outweighs the channel spread (measured -3 % rotated).
  // (Summation order changes with the start; the result is still one fp32 accumulation per
  // element.)  Not applied when the last stage is ragged.
  const int rot = (A_KC || ragged) ? 0 : (int)(((unsigned)(blockIdx.x & 7) * (unsigned)KT) / 8u);
  auto stage_at = [&](int t) {   // t-th stage of the walk (t < KT)
    int e = t + rot;
    if (e >= KT) e -= KT;
    return e;
  };

  TileRef cur_tile = locate_tile<A_KC, B_KC>(p, v, tiles_m, tiles_n);

  // Requests stages first .. NS-2 of `tile` and the A part of stage NS-1 (its B part is the first
  // thing the loop requests); stage t goes to the slot t places after `slot0`.
  auto fill_ring = [&](const Loader<A_KC>& la, const Loader<B_KC>& lb, int lane, const TileRef& tile, uint32_t slot0, int first) {
#pragma unroll
    for (int t = 0; t < NS; ++t) {
      if (t < first) continue;
      uint32_t slot = slot0 + (uint32_t)t * STAGE;
      if (slot >= lds + NS * STAGE) slot -= NS * STAGE;
      const bool tail = (t == KT - 1) && ragged;
      const uint32_t soa = t < KT ? tile.offa + (uint32_t)stage_at(t) * kstep_a : OOB;
      const uint32_t sob = t < KT ? tile.offb + (uint32_t)stage_at(t) * kstep_b : OOB;
#pragma unroll
      for (int i = 0; i < 4; ++i) la.issue_one(ra, slot, wave, lane, soa, i, tail, krem);
      if (t < NS - 1) {
#pragma unroll
        for (int i = 0; i < 4; ++i) lb.issue_one(rb, slot + REGION, wave, lane, sob, i, tail, krem);
      }
    }
  };

  // Loop-carried scalars: LDS slots of stage kt-1 (prv) and kt (cur).  Loads of one stage are
  // split over two phases: its A part in phase 1 of iteration kt (stage kt+NS into slot cur), its
  // B part in phase 0 of iteration kt+1 (same stage, same slot, by then called prv).
  uint32_t cur = lds, prv = lds + (NS - 1) * STAGE;
  const uint32_t wave_lds = (uint32_t)wave * 4096u;   // this wave's 4 KiB share of an operand region

  bool first_tile = true;
  for (;;) {
    // Per-lane addressing state, derived for every tile from a lane id the compiler cannot see
    // through and scoped to the tile: none of it may stay live across the epilogue, which needs
    // every register it can get for the 256 accumulators.
    Loader<A_KC> la;
    Loader<B_KC> lb;
    FragReader<A_KC> fa;
    FragReader<B_KC> fb;
    const int lane = lane_id();
    la.init(wave, lane, 0, lda);
    lb.init(wave, lane, 0, ldb);
    fa.init(lane, wm0);
    fb.init(lane, wn0);
    // ---- the tile's ring: everything for the first tile and without the overlap (wait for
    //      stage 0 only); else stages 0 .. NS-3 landed before the previous epilogue ----
    if (first_tile || !overlap) {
      fill_ring(la, lb, lane, cur_tile, cur, 0);
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" : : "i"(8 * (NS - 2) + 4) : "memory");
    } else {
      fill_ring(la, lb, lane, cur_tile, cur, NS - 2);
    }
    first_tile = false;
    SRT_FENCE();

    const int vn = v + grid;
    const bool has_next = vn < total;
    const TileRef next_tile = locate_tile<A_KC, B_KC>(p, has_next ? vn : v, tiles_m, tiles_n);
    const bool prefetch = overlap && has_next;

    // acc[i][j] is the transposed 32 x 32 tile: m = 32 i + lane % 32, n = 32 j + 8 (v/4) + 4 (lane/32) + v % 4
    f32x16_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    u32x4_t af[2][4], bf[2][4];   // [k slice][32-wide tile]
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      af[0][t] = fa.read(cur, t, 0);
      bf[0][t] = fb.read(cur + REGION, t, 0);
    }

    // The loop body is branch-free.  A request past the tile's last stage is either a stage of
    // the next tile (the first NS - 2 of them, when the overlap is on) or aimed out of range: it
    // returns zeros without touching memory and lands in a slot nobody reads before it is
    // refilled -- those requests are still issued so that the count of loads in flight, which
    // the waits below rely on, is the same in every iteration.
    // Request r (r-th stage counted from this tile's first) reads stage (r + rot) mod KT of its
    // tile -- the same expression for this tile's stages and the next one's -- at the tile's
    // base offset, through the tile's descriptor.  Iteration kt requests the A part of r = kt + NS
    // in its phase 1 and iteration kt + 1 the B part of the same r in its phase 0, so the scalars
    // of both are worked out together, in the shadow of phase 0's MFMAs, from a stage counter
    // that is advanced by one per iteration (no multiplications, no branches).
    const int limit = prefetch ? KT + NS - 2 : KT;   // requests below this index are real
    auto stage_of = [&](int r) {
      int e = r + rot;
      e = e >= KT ? e - KT : e;
      e = e >= KT ? e - KT : e;
      return e;
    };
    uint32_t sob, soa = 0;
    sob = NS - 1 < KT ? cur_tile.offb + (uint32_t)stage_of(NS - 1) * kstep_b : OOB;   // B part of r = NS - 1
    int e_req = stage_of(NS);                                                         // stage of r = NS
    uint32_t ea_off = (uint32_t)e_req * kstep_a, eb_off = (uint32_t)e_req * kstep_b;
    // The loop exists twice: the copy for a ragged last k stage also aims the chunks at or beyond
    // K out of range when that stage is requested (a dozen instructions per trip that the
    // common case does without).
    auto k_loop = [&](auto ragged_tag) {
    constexpr bool RAGGED = decltype(ragged_tag)::value;
    for (int kt = 0; kt < KT; ++kt) {
      uint32_t nxt = cur + STAGE;
      if (nxt == lds + NS * STAGE) nxt = lds;

      // ---- phase 0: MFMAs of slice 0.  The eight fragment reads of slice 1 ride on the first
      //      eight MFMAs so that they have returned by the time the barrier is reached; the B part
      //      of stage kt-1+NS rides on the second eight. ----
      const int kb = kt - 1 + NS;
      const int ka = kt + NS;
      uint32_t sob_next = OOB;
      if (RAGGED) {   // the requests of this iteration that fetch the ragged last stage
        if (kb == KT - 1) lb.mask_tail(wave, lane, krem);
        if (ka == KT - 1) la.mask_tail(wave, lane, krem);
      }
      const uint32_t b_target = prv + REGION + wave_lds;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int u = i * 4 + j;   // 0..15
          if (u == 8) set_lds_target<0>(b_target);
          if (u == 10) set_lds_target<1024>(b_target);
          if (u == 12) set_lds_target<2048>(b_target);
          if (u == 14) set_lds_target<3072>(b_target);
          if (u >= 8 && (u & 1) == 0) SRT_FENCE();
          acc[i][j] = mfma<T>(bf[0][j], af[0][i], acc[i][j]);
          pin(acc[i][j]);
          if (u >= 8 && (u & 1) == 0) {
            SRT_FENCE();
            load_to_lds_at_m0(rb, lb.voff[(u - 8) >> 1], sob);
          }
          // order of first use in phase 1: a0 b0 b1 b2 b3 a1 a2 a3
          if (u == 0) af[1][0] = fa.read(cur, 0, 1);
          else if (u >= 1 && u <= 4) bf[1][u - 1] = fb.read(cur + REGION, u - 1, 1);
          else if (u >= 5 && u <= 7) af[1][u - 4] = fa.read(cur, u - 4, 1);
          // scalars of request r = ka (A part now, B part in the next iteration), a few per MFMA
          if (u == 2) soa = ka < limit ? (ka < KT ? cur_tile.offa : next_tile.offa) + ea_off : OOB;
          if (u == 3) sob_next = ka < limit ? (ka < KT ? cur_tile.offb : next_tile.offb) + eb_off : OOB;
          if (u == 6) {
            const bool wrap = e_req + 1 == KT;
            e_req = wrap ? 0 : e_req + 1;
            ea_off = wrap ? 0u : ea_off + kstep_a;
            eb_off = wrap ? 0u : eb_off + kstep_b;
          }
          SRT_FENCE();
        }
      }

      // ---- sync: all of stage kt is in registers, stage kt+1 has landed ----
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" : : "i"(8 * (NS - 2)) : "memory");
      SRT_FENCE();

      // ---- phase 1: MFMAs of slice 1; the A part of stage kt+NS goes into the slot just vacated
      //      (even MFMAs 0..6), the reads of slice 0 of stage kt+1 ride on the odd MFMAs ----
      const uint32_t a_target = cur + wave_lds;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int u = i * 4 + j;   // 0..15
          if (u == 0) set_lds_target<0>(a_target);
          if (u == 2) set_lds_target<1024>(a_target);
          if (u == 4) set_lds_target<2048>(a_target);
          if (u == 6) set_lds_target<3072>(a_target);
          if (u < 8 && (u & 1) == 0) SRT_FENCE();
          acc[i][j] = mfma<T>(bf[1][j], af[1][i], acc[i][j]);
          pin(acc[i][j]);
          if (u < 8 && (u & 1) == 0) {
            SRT_FENCE();
            load_to_lds_at_m0(ra, la.voff[u >> 1], soa);
          }
          if (u & 1) {
            const int r = u >> 1;   // 0..7, same first-use order as above
            if (r == 0) af[0][0] = fa.read(nxt, 0, 0);
            else if (r <= 4) bf[0][r - 1] = fb.read(nxt + REGION, r - 1, 0);
            else af[0][r - 4] = fa.read(nxt, r - 4, 0);
          }
          SRT_FENCE();
        }
      }
      prv = cur;
      cur = nxt;
      sob = sob_next;
    }
    };
    if (ragged) k_loop(std::true_type{});
    else k_loop(std::false_type{});
    // Every load in flight must have landed, in every wave, before the slots vacated last become
    // the staging area (the out-of-range fillers write zeros there); with the overlap on this
    // also covers the next tile's first stages.
    const int em0 = cur_tile.m0 + wm0, en0 = cur_tile.n0 + wn0, bz = cur_tile.bz;
    // the epilogue's per-lane address arithmetic starts from a lane id the compiler cannot see
    // through: otherwise it is hoisted out of the tile loop and held (spilled) across the k loop
    const int le = lane_id();
    constexpr bool LINEAR_BIAS = EPI == EPI_BIAS || EPI == EPI_BIAS_RELU || EPI == EPI_CLIPPED;
    u32x2_t bias_regs[16];
    if (LINEAR_BIAS) load_bias<T>(p, em0, en0, le, bias_regs);   // lands during the wait below
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (LINEAR_BIAS) pin_all(acc);   // no copy out of the accumulators is scheduled ahead of the wait (registers stay free for the bias)
    // staging: waves 0, 1 share the slot of stage KT-2, waves 2, 3 the slot of stage KT-1
    uint32_t pprv = prv - STAGE;
    if (prv == lds) pprv = lds + (NS - 1) * STAGE;
    const uint32_t stage = ((wave & 2) ? prv : pprv) + (uint32_t)(wave & 1) * 16384u;

    // ---- epilogue ----
    if (EPI == EPI_TRANS) {
      load_bias<T>(p, em0, en0, le, bias_regs);   // one round of latency, before any store is in flight
      store_tile_transcendental<T>(p, acc, em0, en0, bz, le, stage, bias_regs);
    } else {
      store_tile_linear<T, EPI>(p, acc, em0, en0, bz, le, stage, bias_regs);
    }
    if (!has_next) break;

    // ---- next tile: the rest of its ring.  Every wave has finished reading its staging area
    //      before any wave's loads overwrite it. ----
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    v = vn;
    cur_tile = next_tile;
  }
}

#undef SRT_FENCE

// Host-side preconditions beyond those of the MFMA family: every operand tensor (all
// batches) must span less than 1 Gi elements so 32-bit byte offsets reach it (including the rows
// of a partial last tile), and C
// must take aligned 16-byte stores of eight whole columns.
inline bool ring_fits(const GemmProblem& p, bool a_kc, bool b_kc) {
  const long long lda = a_kc ? p.sam : p.sak, ldb = b_kc ? p.sbn : p.sbk;
  const long long nb = p.batch - 1;
  const long long a_reach = nb * p.sab + (a_kc ? ((long long)p.M + BM) * lda + p.K : ((long long)p.K + BK) * lda + p.M + BM);
  const long long b_reach = nb * p.sbb + (b_kc ? ((long long)p.N + BN) * ldb + p.K : ((long long)p.K + BK) * ldb + p.N + BN);
  const long long c_reach = ((long long)p.M + BM) * p.scm + p.N + BN;
  const long long lim = 0x7fffffffLL / 2 - 4096;   // in elements: byte offsets stay below 2^31
  if (!(a_reach < lim && b_reach < lim && c_reach < lim)) return false;
  if (p.sab < 0 || p.sbb < 0) return false;
  if ((p.N % 8) != 0 || (p.scm % 8) != 0 || (p.scb % 8) != 0) return false;
  if ((reinterpret_cast<uintptr_t>(p.C) & 15u) != 0) return false;
  return true;
}

// Workgroups of the persistent grid: one per compute unit (a workgroup takes a whole unit's LDS),
// a multiple of 8 because the XCD-aware tile order wants the stride between a workgroup's tiles
// to be one -- and, when the tiles do not fill the last round, only as many as spread them evenly
// over the same number of rounds (688 tiles: 232 workgroups of 3 tiles instead of 176 with 3 and
// 80 with 2).  Worth 2 % on that shape (276 -> 271 us): units that idle through a ragged last
// round give nothing back, and fewer units per round contend less for L2 and fabric.
inline int persistent_grid(long long tiles) {
  int grid = compute_units() & ~7;
  if (grid <= 0) grid = 8;
  if (tiles < grid) return (int)tiles;
  const long long rounds = (tiles + grid - 1) / grid;
  const long long even = ((tiles + rounds - 1) / rounds + 7) & ~7LL;
  return even < grid ? (int)even : grid;
}

template <typename T, bool A_KC, bool B_KC, int EPI, int NS>
hipError_t launch_kernel(const GemmProblem& p, hipStream_t stream) {
  auto kernel = gemm_ring_kernel<T, A_KC, B_KC, EPI, NS>;
  constexpr int lds_bytes = NS * STAGE;
  static std::atomic<uint32_t> configured{0};
  if (hipError_t e = ensure_lds_limit(reinterpret_cast<const void*>(kernel), lds_bytes, configured); e != hipSuccess) return e;
  const long long tiles = (long long)((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN) * p.batch;
  // one workgroup per compute unit (a workgroup takes a whole unit's LDS); the XCD-aware tile
  // order wants the stride between a workgroup's tiles to be a multiple of 8
  const int grid = persistent_grid(tiles);
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(NT), lds_bytes, stream, p);
  return launch_status(stream);
}

template <typename T, bool A_KC, bool B_KC, int NS = 5>
hipError_t launch(const GemmProblem& p, hipStream_t stream) {
  const bool trans = p.activation == srtActivationSigmoid || p.activation == srtActivationTanh ||
                     p.activation == srtActivationElu;
  if (trans) return launch_kernel<T, A_KC, B_KC, EPI_TRANS, NS>(p, stream);
  if (p.activation == srtActivationClippedRelu) return launch_kernel<T, A_KC, B_KC, EPI_CLIPPED, NS>(p, stream);
  if (p.activation == srtActivationRelu) {
    if (p.bias) return launch_kernel<T, A_KC, B_KC, EPI_BIAS_RELU, NS>(p, stream);
    return launch_kernel<T, A_KC, B_KC, EPI_RELU, NS>(p, stream);
  }
  if (p.bias) return launch_kernel<T, A_KC, B_KC, EPI_BIAS, NS>(p, stream);
  return launch_kernel<T, A_KC, B_KC, EPI_PLAIN, NS>(p, stream);
}

}  // namespace ring
}  // namespace srt
