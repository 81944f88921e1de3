// 256 x 256 bf16 / fp16 matmul tile kernel for gfx950 on v_mfma_f32_16x16x32: the persistent,
// direct-to-LDS ring of gemm_mfma_ring.h (same stage layout, tile walk and cross-tile prefetch --
// see there; swizzles of its own) with the 128 x 128 wave tile cut into 8 x 8 MFMA tiles of 16 x 16
// instead of 4 x 4 tiles of 32 x 32.
//
// Why a second instruction shape.  On N(0,1) data this part runs against its power limit, and
// what a GEMM sustains is set by the energy it spends per flop.  A loop of nothing but MFMAs on
// such data, all CUs, four waves each with 256 accumulator registers per lane:
//     32x32x16                         1780-1800 TFLOP/s
//     16x16x32                         2050      TFLOP/s
// and with the LDS fragment reads a 128 x 128 wave tile needs (16 KiB per wave and k = 32):
//     32x32x16, 16 reads / 32 MFMAs    1575-1585 TFLOP/s
//     16x16x32, 16 reads / 64 MFMAs    1720      TFLOP/s
// Both shapes read the same fragment bytes per flop; the 16x16x32 instruction itself is the
// cheaper one.
//
// The MFMAs are written as inline assembly with the accumulator tile as a tied in/out operand.
// Given the builtin, the register allocator does not keep source and destination accumulator in
// the same registers once all 256 accumulator registers are live: it rotates tiles through
// spare registers with v_accvgpr moves between the MFMAs (measured on an MFMA-only loop: 1760
// instead of 2435 TFLOP/s on zeros).  The compiler does not know the statement is an MFMA, so the
// wait states the hardware needs between an MFMA and a dependent non-MFMA access of its
// accumulator are written out where they could matter (after the k loop).
//
// An MFMA operand is 16 rows x 32 k: lane l holds row l % 16, k = 8 (l / 16) .. + 7 -- one
// ds_read_b128 from a k-contiguous region, two ds_read_b64_tr_b16 from an mn-contiguous one.
// The MFMA takes the B fragment first, so a 16 x 16 accumulator tile is C^T: lane l owns row
// m = l % 16 and the four consecutive columns n = 4 (l / 16) .. + 3.
//
// Pipeline per stage and wave (two phases of 32 MFMAs, 16 cycles each):
//   phase 0   MFMAs of A tiles 0-3 x B tiles 0-7; the reads of B tiles 4-7 and A tiles 4-7 ride on
//             the first half, the four B loads of stage s-1+NS on the second
//   sync      s_waitcnt vmcnt(8 (NS-2)) lgkmcnt(0); s_barrier -- stage s+1 has landed for every
//             wave, every wave holds all of stage s in registers: its slot is free
//   phase 1   MFMAs of A tiles 4-7, with the four A loads of stage s+NS and the reads of stage
//             s+1 (A and B tiles 0-3, B tile j as soon as its last MFMA of the stage has issued)
#pragma once
#include "gemm_mfma_ring.h"

namespace srt {
namespace m16 {

using ring::bf16x8_t;
using ring::f16x8_t;
using ring::f32x4_t;
using ring::u32x2_t;
using ring::u32x4_t;
using ring::s16x4_t;
using ring::BK;
using ring::BN;
using ring::NT;
using ring::OOB;
using ring::REGION;
using ring::STAGE;
using ring::TileRef;
using ring::EPI_PLAIN;
using ring::EPI_BIAS;
using ring::EPI_RELU;
using ring::EPI_BIAS_RELU;
using ring::EPI_CLIPPED;
using ring::EPI_TRANS;
constexpr int EPI_PARTIAL = 6;   // fp32 accumulators as they are, for a split-K pass (C is a float workspace)
// bias, then sigmoid / tanh / elu applied in registers on the way to the staging area (store_tile; the 64-deep kernel):
constexpr int EPI_SIGMOID = 7, EPI_TANH = 8, EPI_ELU = 9;

#define SRT_FENCE() __builtin_amdgcn_sched_barrier(0)

// acc += b x a (operands are 16 x 32 fragments, the accumulator a 16 x 16 fp32 tile in AGPRs)
template <typename T>
__device__ __forceinline__ void mfma16(f32x4_t& acc, const u32x4_t& b, const u32x4_t& a);
template <>
__device__ __forceinline__ void mfma16<BF16>(f32x4_t& acc, const u32x4_t& b, const u32x4_t& a) {
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(b), "v"(a));
}
template <>
__device__ __forceinline__ void mfma16<F16>(f32x4_t& acc, const u32x4_t& b, const u32x4_t& a) {
  asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(b), "v"(a));
}

// acc = b x a: the first MFMA of a tile takes the constant 0 as its addend, which saves zeroing the
// 256 accumulator registers of every tile (and the wait states between that and the first MFMA)
template <typename T>
__device__ __forceinline__ void mfma16_first(f32x4_t& acc, const u32x4_t& b, const u32x4_t& a);
template <>
__device__ __forceinline__ void mfma16_first<BF16>(f32x4_t& acc, const u32x4_t& b, const u32x4_t& a) {
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=a"(acc) : "v"(b), "v"(a));
}
template <>
__device__ __forceinline__ void mfma16_first<F16>(f32x4_t& acc, const u32x4_t& b, const u32x4_t& a) {
  asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=a"(acc) : "v"(b), "v"(a));
}

// An empty statement that "rewrites" every accumulator tile: reads of the accumulators that follow it in
// the source cannot be scheduled ahead of it (see ring::pin).
template <int TM, int TN = 8>
__device__ __forceinline__ void pin_all(f32x4_t (&acc)[TM][TN]) {
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) asm volatile("" : "+a"(acc[i][j]));
}

// ---- global -> LDS --------------------------------------------------------------------------------
// The ring kernel's loader (four loads per wave, operand and stage; lane l of a load lands at
// LDS byte M0 + 16 l, so the swizzle is applied on the global side) with the swizzles that make
// 16 x 32 fragment reads free of bank conflicts.  The ring kernel's own do not: its k-contiguous
// swizzle (row >> 2) & 3 costs a 16-row ds_read_b128 4 extra cycles (8.0 against 4.75 per
// instruction at full LDS load), and its mn-contiguous one puts the four 16-lane groups of a
// ds_read_b64_tr_b16, which come from k rows 8 g .. 8 g + 3, on the same banks for every g.
//   k-contiguous:  [256 rows][4 chunks of 16 B], chunk c of row r at position c ^ ((r >> 1) & 3)
//   mn-contiguous: [32 k][32 chunks of 16 B], chunk c of k row k at c ^ ((k & 3) << 2) ^ (((k >> 3) & 1) << 1)
// LPW: loads per wave, operand and stage -- 4 for a 256-wide region, 2 for a 128-row k-contiguous one.
template <bool KC, int LPW = 4>
struct Loader {
  static_assert(LPW == 4 || (KC && LPW == 2), "an mn-contiguous region is 256 wide");
  uint32_t voff[LPW];

  // ld: elements between rows (KC) or between k (MN)
  __device__ __forceinline__ void init(int wave, int lane, long long ld) {
    if constexpr (KC) {
      // load i of this wave covers tile rows (wave*LPW + i)*16 .. +15, 4 lanes per 64-byte row
#pragma unroll
      for (int i = 0; i < LPW; ++i) {
        const int row = (wave * LPW + i) * 16 + (lane >> 2);
        const int chunk = (lane & 3) ^ ((row >> 1) & 3);
        voff[i] = (uint32_t)(((long long)row * ld + chunk * 8) * 2);
      }
    } else {
      // load i covers k rows (wave*4 + i)*2 .. +1, 32 lanes per 512-byte k row
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int krow = (wave * 4 + i) * 2 + (lane >> 5);
        const int chunk = (lane & 31) ^ ((krow & 3) << 2) ^ (((krow >> 3) & 1) << 1);
        voff[i] = (uint32_t)(((long long)krow * ld + chunk * 8) * 2);
      }
    }
  }

  // does load i of this lane fetch k values at or beyond K in a ragged last stage of krem values?
  __device__ __forceinline__ bool beyond_k(int wave, int lane, int i, int krem) const {
    if constexpr (KC) {
      const int chunk = (lane & 3) ^ ((lane >> 3) & 3);   // (row >> 1) & 3 depends on the lane only
      return chunk >= (krem + 7) / 8;
    } else {
      return (wave * 4 + i) * 2 + (lane >> 5) >= krem;
    }
  }

  // Load i of this wave for the k stage at scalar byte offset `soff` (or OOB: the load reads zeros
  // without touching memory) into the operand region at LDS address `region`; `tail`: a ragged
  // last stage holding only `krem` k values, what lies at or beyond K must read as zero.
  __device__ __forceinline__ void issue_one(u32x4_t rsrc, uint32_t region, int wave, int lane, uint32_t soff, int i,
                                            bool tail, int krem) const {
    uint32_t v = voff[i];
    if (tail && beyond_k(wave, lane, i, krem)) v = OOB;
    ring::load_to_lds(rsrc, region + (uint32_t)(wave * LPW + i) * 1024u, v, soff);
  }

  // aims what lies at or beyond K out of range for good (the state is derived afresh per tile)
  __device__ __forceinline__ void mask_tail(int wave, int lane, int krem) {
#pragma unroll
    for (int i = 0; i < LPW; ++i)
      if (beyond_k(wave, lane, i, krem)) voff[i] = OOB;
  }
};

// ---- LDS -> MFMA operands: 16 rows x 32 k -------------------------------------------------------
template <bool KC>
struct FragReader {
  uint32_t off[KC ? 1 : 8];   // KC: tile t adds t * 1024; MN: one offset per tile (the swizzle is an XOR)

  // wave_row0: first m (n) of the wave's slice inside the tile (a multiple of 128)
  __device__ __forceinline__ void init(int lane, int wave_row0) {
    const int g = lane >> 4, jn = lane & 15;
    if constexpr (KC) {
      const int f = (jn >> 1) & 3;   // (row >> 1) & 3 for rows wave_row0 + 16 t + jn
      off[0] = (uint32_t)((wave_row0 + jn) * 64 + ((g ^ f) << 4));
    } else {
      // lane supplies the address of T[k = 8 g + e (+ 4 for the second read)][mn = wave_row0 + 16 t + 4 q]
      const int e = jn >> 2, q = jn & 3;
      const int krow = 8 * g + e;
      const int mn = wave_row0 + 4 * q;   // tile t adds 16: two 16-byte chunks
      const uint32_t base = (uint32_t)(krow * 512 + ((mn >> 2) & 1) * 8);
      const int chunk0 = mn >> 3, swz = (e << 2) ^ ((g & 1) << 1);   // k & 3 = e, bit 3 of k = g & 1
#pragma unroll
      for (int t = 0; t < 8; ++t) off[t] = base + (uint32_t)(((chunk0 + 2 * t) ^ swz) << 4);
    }
  }
  __device__ __forceinline__ u32x4_t read(uint32_t region, int t) const {
    if constexpr (KC) {
      return *reinterpret_cast<const SRT_LDS u32x4_t*>(region + off[0] + t * 1024);
    } else {
      const uint32_t a = region + off[t];
      const u32x2_t lo =
          __builtin_bit_cast(u32x2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<SRT_LDS s16x4_t*>(a)));
      const u32x2_t hi = __builtin_bit_cast(
          u32x2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<SRT_LDS s16x4_t*>(a + 2048)));
      u32x4_t v = {lo.x, lo.y, hi.x, hi.y};
      return v;
    }
  }
};

// ---- epilogue ------------------------------------------------------------------------------------
// acc[i][j] is a transposed 16 x 16 tile: lane l owns row m = wave_m0 + 16 i + l % 16 and the
// columns n = wave_n0 + 16 j + 4 (l / 16) + 0..3.
//
// The bias values a lane adds -- 32 per-column ones (or TM per-row ones after a C^T flip) -- are
// requested in one batch right after the k loop, ahead of the wait and barrier that end it, so
// their latency passes while the matrix pipe drains.  Read where they are used, inside the pass
// over the accumulators, they came in eight dependent rounds of a global load's latency each
// (5.5 us of a 95 us tile at K = 4096).  A dense, 8-byte-aligned bias is read as eight 8-byte loads.
// They wait in their stored 16-bit form, two to a register (16 registers per lane): b[j] holds the four
// per-column values of column tile j; in the per-row case b[i].x holds row tile i's value.
template <typename T, int TM>
__device__ __forceinline__ void load_bias(const GemmProblem& p, int wave_m0, int wave_n0, int lane, u32x2_t (&b)[8]) {
  using S = typename T::storage;
  static_assert(sizeof(S) == 2 && TM <= 8, "16-bit element types, at most 8 row tiles");
  const S* bias = (const S*)p.bias;
  const int jn = lane & 15, g = lane >> 4;
#pragma unroll
  for (int j = 0; j < 8; ++j) b[j] = u32x2_t{0u, 0u};
  if (!bias) return;
  if (p.bias_per_row) {
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int m = wave_m0 + 16 * i + jn;
      if (m < p.M) b[i].x = bias[(long long)m * p.sbias];
    }
  } else if (p.sbias == 1 && (reinterpret_cast<uintptr_t>(bias) & 7u) == 0) {
    // N is a multiple of 8 and n of 4: a lane's four columns are all inside or all outside
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int n = wave_n0 + 16 * j + 4 * g;
      if (n < p.N) b[j] = *reinterpret_cast<const u32x2_t*>(bias + n);
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      uint32_t h[4] = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int n = wave_n0 + 16 * j + 4 * g + e;
        if (n < p.N) h[e] = bias[(long long)n * p.sbias];
      }
      b[j] = u32x2_t{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
    }
  }
}

// One rounding to the element type, then a trip through the wave's staging area at LDS address
// `stage` so that global stores are whole 16-byte chunks of 256-byte row segments.  Passes of ROWS
// rows (64: 16 KiB of staging, the 128-row wave tile; 32: 8 KiB, the 64-row one):
// [ROWS rows][16 chunks of 16 B], chunk c of row r at position c ^ (r & 15) (conflict-free on both
// sides: a write instruction covers 16 rows x 32 B, a read 4 whole rows).
// NaN handling as in ring::store_tile: the hardware converter rounds everything, and when any
// lane of the wave saw a NaN the staged patterns are rewritten to 0x7FFF on the way out.
// Bias and the activation (CLAMP 1: relu, 2: clipped relu, 3: sigmoid, 4: tanh, 5: elu) are applied to the copy that
// leaves the accumulator registers, so the accumulators themselves are only read.  The transcendental ones are
// straight-line code per value (activation16_ct: selects, no branches) -- 256 copies of a dozen instructions per
// lane, fetched once per tile.  Against staging fp32 values and applying the activation in a rolled loop
// (store_tile_transcendental) that saves the second trip through LDS, the scalar encoder and the 8-byte stores:
// 4096 x 8192 x 4096 + bias + tanh 213-220 us that way, 181 plain.
// FLIP: the accumulator of the tile in row group i, column group j of the result is acc[j][i] (the kernel computed
// the transposed product with the operands' roles exchanged; each 16 x 16 tile lies in the registers as it does
// otherwise).
// TN: column tiles per wave (8; 6 for the 192-wide workgroup tile, whose wave covers 96 columns).  n_end: columns at
// or beyond it belong to another tile and are not stored (a workgroup tile narrower than its MFMA footprint).
template <typename T, int TM, bool HAS_BIAS, int CLAMP, bool FLIP = false, int TN = 8>
__device__ __forceinline__ void store_tile(const GemmProblem& p, const f32x4_t (&acc)[TM][TN], int wave_m0, int wave_n0,
                                           int bz, int lane, uint32_t stage, const u32x2_t (&b)[8], int n_end = 0x7fffffff) {
  static_assert(!FLIP || (TM == 8 && TN == 8), "a square block of accumulator tiles");
  static_assert(TN <= 8, "the staging rows hold 16 chunks");
  constexpr int ROWS = TM == 8 ? 64 : 32;
  using S = typename T::storage;
  const bool per_row = p.bias_per_row != 0;
  const float ceiling = p.coef;
  constexpr bool FIXUP = T::dtype == srtReal16BF;
  S* C = (S*)p.C + (long long)bz * p.scb;
  const long long c_last = (long long)(p.M - 1) * p.scm + p.N;
  const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc(C, 0, (int)(c_last * 2), 0x00020000);
  const int ldc2 = (int)(p.scm * 2);
  const int jn = lane & 15, g = lane >> 4;
  const int rd_chunk = lane & 15, rd_row = lane >> 4;   // read side: chunk of rows rd_row + 4 it
  const int n_rd = wave_n0 + 8 * rd_chunk;
  // N is a multiple of 8 (checked on the host): the chunk is whole
  const bool n_rd_ok = n_rd < p.N && (TN == 8 || (rd_chunk < 2 * TN && n_rd < n_end));

  // staging address of accumulator tile (ii, j): row 16 ii + jn, chunk (2 j + g / 2) ^ jn -- the lane's part of
  // it is the same for every ii (a row group is 4096 bytes further: an immediate offset of the write)
  uint32_t wr[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j)
    wr[j] = stage + (uint32_t)jn * 256u + (uint32_t)(g & 1) * 8u + (uint32_t)(((2 * j + (g >> 1)) ^ jn) << 4);

#pragma unroll
  for (int half = 0; half < TM * 16 / ROWS; ++half) {
    bool nan = false;
#pragma unroll
    for (int ii = 0; ii < ROWS / 16; ++ii) {
      const int i = (ROWS / 16) * half + ii;
      SRT_FENCE();
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        float a0, a1, a2, a3;
        if constexpr (FLIP) { a0 = acc[j][i][0]; a1 = acc[j][i][1]; a2 = acc[j][i][2]; a3 = acc[j][i][3]; }
        else { a0 = acc[i][j][0]; a1 = acc[i][j][1]; a2 = acc[i][j][2]; a3 = acc[i][j][3]; }
        if (HAS_BIAS) {
          const float br = T::to_float((S)(b[i].x & 0xffffu));
          a0 += per_row ? br : T::to_float((S)(b[j].x & 0xffffu));
          a1 += per_row ? br : T::to_float((S)(b[j].x >> 16));
          a2 += per_row ? br : T::to_float((S)(b[j].y & 0xffffu));
          a3 += per_row ? br : T::to_float((S)(b[j].y >> 16));
        }
        if (CLAMP == 1 || CLAMP == 2) {
          a0 = __builtin_fmaxf(a0, 0.0f); a1 = __builtin_fmaxf(a1, 0.0f);
          a2 = __builtin_fmaxf(a2, 0.0f); a3 = __builtin_fmaxf(a3, 0.0f);
        }
        if (CLAMP == 2) {
          a0 = __builtin_fminf(a0, ceiling); a1 = __builtin_fminf(a1, ceiling);
          a2 = __builtin_fminf(a2, ceiling); a3 = __builtin_fminf(a3, ceiling);
        }
        if (CLAMP >= 3) {
          constexpr int ACT = CLAMP == 3 ? srtActivationSigmoid : CLAMP == 4 ? srtActivationTanh : srtActivationElu;
          a0 = activation16_ct<ACT>(ceiling, a0); a1 = activation16_ct<ACT>(ceiling, a1);
          a2 = activation16_ct<ACT>(ceiling, a2); a3 = activation16_ct<ACT>(ceiling, a3);
        }
        if (FIXUP) nan |= __builtin_isunordered(a0, a1) | __builtin_isunordered(a2, a3);
        const u32x2_t w = {T::template pack2<false>(a0, a1), T::template pack2<false>(a2, a3)};
        *reinterpret_cast<SRT_LDS u32x2_t*>(wr[j] + (uint32_t)ii * 4096u) = w;
      }
    }
    SRT_FENCE();
    const bool fix = FIXUP && __builtin_amdgcn_ballot_w64(nan) != 0;
    // ---- staging -> global: ROWS / 4 instructions of 4 rows x 256 bytes, read four at a time ----
#pragma unroll
    for (int it4 = 0; it4 < ROWS / 16; ++it4) {
      u32x4_t v[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int row = rd_row + 4 * (4 * it4 + q);
        v[q] = *reinterpret_cast<const SRT_LDS u32x4_t*>(stage + (uint32_t)row * 256u +
                                                         (uint32_t)((rd_chunk ^ (row & 15)) << 4));
      }
      if (fix) {   // rare: some accumulator of this half was a NaN
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int e = 0; e < 4; ++e) v[q][e] = ring::canonical_nans_bf16x2(v[q][e]);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int row = rd_row + 4 * (4 * it4 + q);
        const int m = wave_m0 + ROWS * half + row;
        const uint32_t off = (n_rd_ok && m < p.M) ? (uint32_t)(m * ldc2 + n_rd * 2) : OOB;
        __builtin_amdgcn_raw_buffer_store_b128(v[q], rc, (int)off, 0, SRT_STORE_AUX);
      }
      SRT_FENCE();
    }
  }
}

// sigmoid / tanh / elu: acc + bias goes to the staging area as fp32 (passes of ROWS = 32 or 16 rows:
// [ROWS rows][32 chunks of 16 B], chunk c of row r at c ^ (r & 31)); activation, rounding and store
// run in a rolled loop.
template <typename T, int TM>
__device__ __forceinline__ void store_tile_transcendental(const GemmProblem& p, const f32x4_t (&acc)[TM][8],
                                                          int wave_m0, int wave_n0, int bz, int lane, uint32_t stage,
                                                          const u32x2_t (&b)[8]) {
  constexpr int ROWS = TM == 8 ? 32 : 16;
  using S = typename T::storage;
  S* C = (S*)p.C + (long long)bz * p.scb;
  const long long c_last = (long long)(p.M - 1) * p.scm + p.N;
  const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc(C, 0, (int)(c_last * 2), 0x00020000);
  const int ldc2 = (int)(p.scm * 2);
  const bool per_row = p.bias_per_row != 0;
  const int jn = lane & 15, g = lane >> 4;
  const int rd_chunk = lane & 31, rd_row = lane >> 5;   // read side: 4 columns of rows rd_row + 2 it
  const int n_rd = wave_n0 + 4 * rd_chunk;
  const bool n_rd_ok = n_rd < p.N;
#pragma unroll
  for (int pass = 0; pass < TM * 16 / ROWS; ++pass) {
#pragma unroll
    for (int ii = 0; ii < ROWS / 16; ++ii) {
      const int i = (ROWS / 16) * pass + ii;
      const int row = 16 * ii + jn;
      // bias from the registers load_bias filled before the tile's first store was issued: a global load
      // in here would wait, with its vmcnt(0), for every store of the previous pass as well
      const float brow = T::to_float((S)(b[i].x & 0xffffu));
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float bcol[4] = {T::to_float((S)(b[j].x & 0xffffu)), T::to_float((S)(b[j].x >> 16)),
                               T::to_float((S)(b[j].y & 0xffffu)), T::to_float((S)(b[j].y >> 16))};
        f32x4_t x;
#pragma unroll
        for (int e = 0; e < 4; ++e) x[e] = acc[i][j][e] + (per_row ? brow : bcol[e]);
        const int c = 4 * j + g;
        *reinterpret_cast<SRT_LDS f32x4_t*>(stage + (uint32_t)row * 512u + (uint32_t)((c ^ (row & 31)) << 4)) = x;
      }
    }
    // the staged values' activation, rounding and store: one copy of the loop per activation, chosen by a
    // uniform branch (a switch per element inside the loop costs a chain of branches each)
    auto tail = [&](auto act) __attribute__((always_inline)) {
      constexpr int ACT = decltype(act)::value;
#pragma unroll 4
      for (int it = 0; it < ROWS / 2; ++it) {
        const int row = rd_row + 2 * it;
        const f32x4_t x = *reinterpret_cast<const SRT_LDS f32x4_t*>(stage + (uint32_t)row * 512u +
                                                                    (uint32_t)((rd_chunk ^ (row & 31)) << 4));
        uint32_t lo = (uint32_t)T::from_float(activation16_ct<ACT>(p.coef, x[0])) |
                      ((uint32_t)T::from_float(activation16_ct<ACT>(p.coef, x[1])) << 16);
        uint32_t hi = (uint32_t)T::from_float(activation16_ct<ACT>(p.coef, x[2])) |
                      ((uint32_t)T::from_float(activation16_ct<ACT>(p.coef, x[3])) << 16);
        const u32x2_t w = {lo, hi};
        const int mm = wave_m0 + ROWS * pass + row;
        const uint32_t off = (n_rd_ok && mm < p.M) ? (uint32_t)(mm * ldc2 + n_rd * 2) : OOB;
        __builtin_amdgcn_raw_buffer_store_b64(w, rc, (int)off, 0, SRT_STORE_AUX);
      }
    };
    if (p.activation == srtActivationSigmoid) tail(std::integral_constant<int, srtActivationSigmoid>{});
    else if (p.activation == srtActivationTanh) tail(std::integral_constant<int, srtActivationTanh>{});
    else tail(std::integral_constant<int, srtActivationElu>{});
    // the rolled loop's reads must have returned before the next pass overwrites the area
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
}

// Split-K pass: the fp32 accumulators go to a float workspace as they are ([batch][M][N], row
// stride scm floats); a second kernel adds the passes and applies the epilogue.  Staged through
// the wave's LDS in passes of ROWS = 32 or 16 rows ([ROWS rows][32 chunks of 16 B], chunk c of row
// r at c ^ (r & 31)) so that a store instruction writes two rows of 512 contiguous bytes: whole
// cache lines (straight from the accumulator layout an instruction would write 16 rows x 64 bytes,
// every line in two halves by different instructions; measured, the two take the same time).
template <int TM>
__device__ __forceinline__ void store_tile_partial(const GemmProblem& p, const f32x4_t (&acc)[TM][8], int wave_m0,
                                                   int wave_n0, int bz, int lane, uint32_t stage) {
  constexpr int ROWS = TM == 8 ? 32 : 16;
  float* C = (float*)p.C + (long long)bz * p.scb;
  const long long c_last = (long long)(p.M - 1) * p.scm + p.N;
  const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc(C, 0, (int)(c_last * 4), 0x00020000);
  const int ldc4 = (int)(p.scm * 4);
  const int jn = lane & 15, g = lane >> 4;
  const int rd_chunk = lane & 31, rd_row = lane >> 5;   // read side: 4 columns of rows rd_row + 2 it
  const int n_rd = wave_n0 + 4 * rd_chunk;
  const bool n_rd_ok = n_rd < p.N;   // N is a multiple of 8: the four columns are in range together
#pragma unroll
  for (int pass = 0; pass < TM * 16 / ROWS; ++pass) {
#pragma unroll
    for (int ii = 0; ii < ROWS / 16; ++ii) {
      const int i = (ROWS / 16) * pass + ii;
      const int row = 16 * ii + jn;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int c = 4 * j + g;
        *reinterpret_cast<SRT_LDS f32x4_t*>(stage + (uint32_t)row * 512u + (uint32_t)((c ^ (row & 31)) << 4)) = acc[i][j];
      }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int it4 = 0; it4 < ROWS / 8; ++it4) {
      f32x4_t v[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int row = rd_row + 2 * (4 * it4 + q);
        v[q] = *reinterpret_cast<const SRT_LDS f32x4_t*>(stage + (uint32_t)row * 512u +
                                                         (uint32_t)((rd_chunk ^ (row & 31)) << 4));
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int row = rd_row + 2 * (4 * it4 + q);
        const int m = wave_m0 + ROWS * pass + row;
        const uint32_t off = (n_rd_ok && m < p.M) ? (uint32_t)(m * ldc4 + n_rd * 4) : OOB;
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, v[q]), rc, (int)off, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // the reads of this pass have returned (their data is in the stores above) before the next
    // pass overwrites the area: LDS operations of a wave execute in order
  }
}

// ring::locate_tile for a tile of TILE_M x 256
template <bool A_KC, bool B_KC, int TILE_M>
__device__ __forceinline__ TileRef locate_tile(const GemmProblem& p, int v, int tiles_m, int tiles_n) {
  const int per_batch = tiles_m * tiles_n;
  const int bz = v / per_batch;
  int tm, tn;
  ring::tile_coords(v - bz * per_batch, tiles_m, tiles_n, &tm, &tn);
  TileRef t;
  t.m0 = tm * TILE_M;
  t.n0 = tn * BN;
  t.bz = bz;
  const long long lda = A_KC ? p.sam : p.sak;
  const long long ldb = B_KC ? p.sbn : p.sbk;
  t.offa = (uint32_t)(((long long)bz * p.sab + (A_KC ? (long long)t.m0 * lda : (long long)t.m0)) * 2);
  t.offb = (uint32_t)(((long long)bz * p.sbb + (B_KC ? (long long)t.n0 * ldb : (long long)t.n0)) * 2);
  return t;
}

// Slot of a phase (MFMA index u) at which an event of the schedule happens, or its index if u is
// such a slot (-1 otherwise).  TM = 8: phases of 32 MFMAs, TM = 4: of 16.
template <int TM> constexpr int phase0_b_read(int u) {      // B tiles 4-7, before their first use at u = 2 TM
  return TM == 8 ? ((u < 8 && (u & 1) == 0) ? u >> 1 : -1) : (u < 4 ? u : -1);
}
template <int TM> constexpr int phase0_a_read(int u) {      // A tiles of phase 1
  return TM == 8 ? ((u >= 8 && u < 16 && (u & 1) == 0) ? (u - 8) >> 1 : -1) : ((u == 4 || u == 5) ? u - 4 : -1);
}
template <int TM> constexpr int phase0_b_load(int u) {      // the four B loads of the stage requested
  return TM == 8 ? ((u >= 16 && (u & 3) == 0) ? (u - 16) >> 2 : -1) : ((u >= 8 && (u & 1) == 0) ? (u - 8) >> 1 : -1);
}
template <int TM> constexpr int phase0_scalar(int u) {      // scalar events 0..6 (TM = 4: 0 and 1 share a slot)
  if (TM == 8) return (u >= 17 && (u & 1) == 1) ? (u - 17) >> 1 : -1;
  switch (u) { case 6: return 0; case 7: return 2; case 9: return 3; case 11: return 4; case 13: return 5; case 15: return 6; default: return -1; }
}
template <int TM> constexpr int phase1_a_load(int u) {      // the TM / 2 A loads of the stage requested
  return TM == 8 ? ((u >= 16 && (u & 3) == 0) ? (u - 16) >> 2 : -1) : ((u == 8 || u == 12) ? (u - 8) >> 2 : -1);
}
template <int TM> constexpr int phase1_a_read(int u) {      // A tiles of the next stage's phase 0
  return TM == 8 ? ((u < 16 && (u & 3) == 1) ? u >> 2 : -1) : ((u == 0 || u == 2) ? u >> 1 : -1);
}
template <int TM> constexpr int phase1_b_read(int u) {      // B tile j < 4, right after its last MFMA of the stage
  return TM == 8 ? ((u < 16 && (u & 3) == 3) ? u >> 2 : -1) : ((u < 8 && (u & 1) == 1) ? u >> 1 : -1);
}
template <int TM> constexpr int phase1_scalar(int u) {      // scalar events 0..3
  return TM == 8 ? ((u >= 17 && u <= 23 && (u & 1) == 1) ? (u - 17) >> 1 : -1)
                 : ((u >= 9 && (u & 1) == 1) ? (u - 9) >> 1 : -1);
}

// TM: 16-row A tiles per wave.  8: the 256 x 256 tile.  4: a 128 x 256 tile (A region of 128 rows,
// k-contiguous A only), for problems that leave compute units idle with the large tile.
template <typename T, bool A_KC, bool B_KC, int EPI, int NS, int TM = 8>
__global__ __launch_bounds__(NT) void gemm_m16_kernel(GemmProblem p) {
  static_assert(NS == 5, "ring depth");   // five stages of 32 KiB are the whole LDS
  static_assert(TM == 8 || (TM == 4 && A_KC), "the 128-row A region is k-contiguous");
  constexpr int TILE_M = 32 * TM;                 // 256 or 128
  constexpr int LPW_A = TM / 2;                   // A loads per wave and stage
  constexpr int REGION_A = TILE_M * BK * 2;       // bytes of the A part of a stage; the B part (REGION) follows it
  constexpr int STAGE_B = REGION_A + REGION;      // bytes of a stage
  constexpr int LOADS = LPW_A + 4;                // loads per wave and stage
  constexpr int HALF = TM / 2;                    // A tiles per phase (a phase is 8 HALF MFMAs)
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[];
  const uint32_t lds = (uint32_t)(uintptr_t)(SRT_LDS unsigned char*)lds_raw;

  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  auto lane_id = []() {
    uint32_t zero = 0;
    asm volatile("" : "+s"(zero));   // opaque: keeps the two instructions where they are written
    return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, zero));
  };
  const int wm0 = (wave >> 1) * (16 * TM), wn0 = (wave & 1) * 128;

  const int tiles_m = (p.M + TILE_M - 1) / TILE_M, tiles_n = (p.N + BN - 1) / BN;
  const int total = tiles_m * tiles_n * p.batch;
  const int grid = (int)gridDim.x;
  int v = (int)blockIdx.x;

  const long long lda = A_KC ? p.sam : p.sak;
  const long long ldb = B_KC ? p.sbn : p.sbk;
  const long long a_view = A_KC ? (long long)(p.M - 1) * lda + p.K : (long long)(p.K - 1) * lda + p.M;
  const long long b_view = B_KC ? (long long)(p.N - 1) * ldb + p.K : (long long)(p.K - 1) * ldb + p.N;
  const u32x4_t ra = ring::make_rsrc(p.A, (uint32_t)(((long long)(p.batch - 1) * p.sab + a_view) * 2));
  const u32x4_t rb = ring::make_rsrc(p.B, (uint32_t)(((long long)(p.batch - 1) * p.sbb + b_view) * 2));
  const uint32_t kstep_a = A_KC ? (uint32_t)(BK * 2) : (uint32_t)(BK * lda * 2);   // bytes per k stage
  const uint32_t kstep_b = B_KC ? (uint32_t)(BK * 2) : (uint32_t)(BK * ldb * 2);
  const int KT = (p.K + BK - 1) / BK;
  const int krem = p.K % BK;   // k values in a ragged last stage (0: the stage is whole)
  const bool ragged = krem != 0;
  const bool overlap = !ragged && KT >= NS;

  const int rot = (A_KC || ragged) ? 0 : (int)(((unsigned)(blockIdx.x & 7) * (unsigned)KT) / 8u);
  auto stage_at = [&](int t) {   // t-th stage of the walk (t < KT)
    int e = t + rot;
    if (e >= KT) e -= KT;
    return e;
  };

  TileRef cur_tile = locate_tile<A_KC, B_KC, TILE_M>(p, v, tiles_m, tiles_n);

  // Requests stages first .. NS-2 of `tile` and the A part of stage NS-1 (its B part is the first
  // thing the loop requests); stage t goes to the slot t places after `slot0`.
  auto fill_ring = [&](const Loader<A_KC, LPW_A>& la, const Loader<B_KC>& lb, int lane, const TileRef& tile,
                       uint32_t slot0, int first) {
#pragma unroll
    for (int t = 0; t < NS; ++t) {
      if (t < first) continue;
      uint32_t slot = slot0 + (uint32_t)t * STAGE_B;
      if (slot >= lds + NS * STAGE_B) slot -= NS * STAGE_B;
      const bool tail = (t == KT - 1) && ragged;
      const uint32_t soa = t < KT ? tile.offa + (uint32_t)stage_at(t) * kstep_a : OOB;
      const uint32_t sob = t < KT ? tile.offb + (uint32_t)stage_at(t) * kstep_b : OOB;
#pragma unroll
      for (int i = 0; i < LPW_A; ++i) la.issue_one(ra, slot, wave, lane, soa, i, tail, krem);
      if (t < NS - 1) {
#pragma unroll
        for (int i = 0; i < 4; ++i) lb.issue_one(rb, slot + REGION_A, wave, lane, sob, i, tail, krem);
      }
    }
  };

  uint32_t cur = lds, prv = lds + (NS - 1) * STAGE_B;
  const uint32_t wave_lds_a = (uint32_t)wave * (LPW_A * 1024u);   // this wave's share of an A region
  const uint32_t wave_lds_b = (uint32_t)wave * 4096u;              // and of a B region

  bool first_tile = true;
  for (;;) {
    // per-lane addressing state, derived per tile and scoped to it (see gemm_ring_kernel)
    Loader<A_KC, LPW_A> la;
    Loader<B_KC> lb;
    FragReader<A_KC> fa;
    FragReader<B_KC> fb;
    const int lane = lane_id();
    la.init(wave, lane, lda);
    lb.init(wave, lane, ldb);
    fa.init(lane, wm0);
    fb.init(lane, wn0);
    if (first_tile || !overlap) {
      fill_ring(la, lb, lane, cur_tile, cur, 0);
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" : : "i"(LOADS * (NS - 2) + LPW_A) : "memory");
    } else {
      fill_ring(la, lb, lane, cur_tile, cur, NS - 2);
    }
    first_tile = false;
    SRT_FENCE();

    const int vn = v + grid;
    const bool has_next = vn < total;
    const TileRef next_tile = locate_tile<A_KC, B_KC, TILE_M>(p, has_next ? vn : v, tiles_m, tiles_n);
    const bool prefetch = overlap && has_next;

    f32x4_t acc[TM][8];   // defined by the MFMAs of the tile's first stage

    u32x4_t af[TM], bf[8];   // the stage's A and B tiles
#pragma unroll
    for (int t = 0; t < 4; ++t) bf[t] = fb.read(cur + REGION_A, t);
#pragma unroll
    for (int t = 0; t < HALF; ++t) af[t] = fa.read(cur, t);

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

    // Both phases walk their 4 x 8 MFMA tiles B tile by B tile (u = 4 j + i), so that in phase 1
    // B tile j is finished with after MFMA 4 j + 3 and its registers can take tile j of the next
    // stage -- one register set per operand is enough.  Tiles 0-3 of both operands are read in
    // phase 1 of the stage before, tiles 4-7 in phase 0 of their own stage.
    // An MFMA occupies the matrix pipe for 16 cycles and the wave issues one instruction every
    // four, so no gap between two MFMAs should hold more than three other instructions.  Fragment
    // reads take the first half of each phase (one every other MFMA), the loads the second half
    // (one every fourth), and the scalar bookkeeping of the requests is dealt out over the odd
    // slots of the second halves, a few instructions each.
    uint32_t b_target = prv + REGION_A + wave_lds_b;   // landing address of the next B request
    auto set_target = [](int idx, uint32_t base) __attribute__((always_inline)) {
      if (idx == 0) ring::set_lds_target<0>(base);
      if (idx == 1) ring::set_lds_target<1024>(base);
      if (idx == 2) ring::set_lds_target<2048>(base);
      if (idx == 3) ring::set_lds_target<3072>(base);
    };
    auto one_stage = [&](auto ragged_tag, auto first_tag, int kt) __attribute__((always_inline)) {
      constexpr bool RAGGED = decltype(ragged_tag)::value;
      constexpr bool FIRST = decltype(first_tag)::value;   // the tile's first stage: accumulators start here
      const int kb = kt - 1 + NS;
      const int ka = kt + NS;
      if (RAGGED) {
        if (kb == KT - 1) lb.mask_tail(wave, lane, krem);
        if (ka == KT - 1) la.mask_tail(wave, lane, krem);
      }
      uint32_t nxt = 0, a_target = 0, sel = 0, sob_next = OOB;
      bool wrap = false;
      // ---- phase 0: the first half of the A tiles ----
#pragma unroll
      for (int j = 0; j < 8; ++j) {
#pragma unroll
        for (int i = 0; i < HALF; ++i) {
          const int u = j * HALF + i;   // 0 .. SLOTS - 1
          const int ld = phase0_b_load<TM>(u);
          if (ld >= 0) {
            set_target(ld, b_target);
            SRT_FENCE();
          }
          if constexpr (FIRST) mfma16_first<T>(acc[i][j], bf[j], af[i]);
          else mfma16<T>(acc[i][j], bf[j], af[i]);
          if (ld >= 0) {
            SRT_FENCE();
            ring::load_to_lds_at_m0(rb, lb.voff[ld], sob);
          }
          // the rest of stage kt: B tiles 4-7 (first used half way through the phase), the A tiles of phase 1
          const int rb_ = phase0_b_read<TM>(u), ra_ = phase0_a_read<TM>(u);
          if (rb_ >= 0) bf[4 + rb_] = fb.read(cur + REGION_A, 4 + rb_);
          if (ra_ >= 0) af[HALF + ra_] = fa.read(cur, HALF + ra_);
          // request r = ka: its A part goes out in phase 1, its B part in phase 0 of the next stage
          const int ev = phase0_scalar<TM>(u);
          if (ev == 0) nxt = cur + STAGE_B;
          if (ev == 1 || (TM == 4 && ev == 0)) nxt = nxt == lds + NS * STAGE_B ? lds : nxt;
          if (ev == 2) sel = ka < KT ? cur_tile.offa : next_tile.offa;
          if (ev == 3) soa = ka < limit ? sel + ea_off : OOB;
          if (ev == 4) sel = ka < KT ? cur_tile.offb : next_tile.offb;
          if (ev == 5) sob_next = ka < limit ? sel + eb_off : OOB;
          if (ev == 6) a_target = cur + wave_lds_a;
          SRT_FENCE();
        }
      }
      // ---- sync: all of stage kt is in registers, stage kt+1 has landed ----
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" : : "i"(LOADS * (NS - 2)) : "memory");
      SRT_FENCE();
      // ---- phase 1: the second half of the A tiles; reads of stage kt+1; A loads of stage kt+NS ----
#pragma unroll
      for (int j = 0; j < 8; ++j) {
#pragma unroll
        for (int i = 0; i < HALF; ++i) {
          const int u = j * HALF + i;   // 0 .. SLOTS - 1
          const int ld = phase1_a_load<TM>(u);
          if (ld >= 0) {
            set_target(ld, a_target);
            SRT_FENCE();
          }
          if constexpr (FIRST) mfma16_first<T>(acc[HALF + i][j], bf[j], af[HALF + i]);
          else mfma16<T>(acc[HALF + i][j], bf[j], af[HALF + i]);
          if (ld >= 0) {
            SRT_FENCE();
            ring::load_to_lds_at_m0(ra, la.voff[ld], soa);
          }
          // stage kt+1: the A tiles of phase 0 (idle since then) and B tiles 0-3, each as it falls free
          const int ra_ = phase1_a_read<TM>(u), rb_ = phase1_b_read<TM>(u);
          if (ra_ >= 0) af[ra_] = fa.read(nxt, ra_);
          if (rb_ >= 0) bf[rb_] = fb.read(nxt + REGION_A, rb_);
          // the stage of request r = ka + 1, and where its B part will land
          const int ev = phase1_scalar<TM>(u);
          if (ev == 0) {
            wrap = e_req + 1 == KT;
            e_req = wrap ? 0 : e_req + 1;
          }
          if (ev == 1) ea_off = wrap ? 0u : ea_off + kstep_a;
          if (ev == 2) eb_off = wrap ? 0u : eb_off + kstep_b;
          if (ev == 3) b_target = cur + REGION_A + wave_lds_b;
          SRT_FENCE();
        }
      }
      prv = cur;
      cur = nxt;
      sob = sob_next;
    };
    // The loop exists twice (ragged / whole last stage) like the ring kernel's; the common one is
    // unrolled by two, which halves the loop's own bookkeeping.
    auto k_loop = [&](auto ragged_tag) __attribute__((always_inline)) {
      constexpr bool RAGGED = decltype(ragged_tag)::value;
      one_stage(ragged_tag, std::true_type{}, 0);
      int kt = 1;
      if (!RAGGED) {
        for (; kt + 1 < KT; kt += 2) {
          one_stage(ragged_tag, std::false_type{}, kt);
          one_stage(ragged_tag, std::false_type{}, kt + 1);
        }
      }
      for (; kt < KT; ++kt) one_stage(ragged_tag, std::false_type{}, kt);
    };
    if (ragged) k_loop(std::true_type{});
    else k_loop(std::false_type{});

    // Every load in flight must have landed, in every wave, before the slots vacated last become
    // the staging area.  The s_nops are the wait states between the last MFMAs and the first
    // reads of their accumulators by other instructions.
    const int em0 = cur_tile.m0 + wm0, en0 = cur_tile.n0 + wn0, bz = cur_tile.bz;
    const int le = lane_id();
    constexpr bool LINEAR_BIAS = EPI == EPI_BIAS || EPI == EPI_BIAS_RELU || EPI == EPI_CLIPPED;
    u32x2_t bias_regs[8];
    if (LINEAR_BIAS) load_bias<T, TM>(p, em0, en0, le, bias_regs);   // lands during the wait below
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier\n\ts_nop 7\n\ts_nop 7" ::: "memory");
    // with the bias loads ahead of the wait the compiler pulled every accumulator read up there too: the
    // accumulators are "rewritten" here so that no read of them is scheduled above the wait states
    if (LINEAR_BIAS) pin_all<TM>(acc);
    // staging: waves 0, 1 share the slot of stage KT-2, waves 2, 3 the slot of stage KT-1 (half a slot each)
    uint32_t pprv = prv - STAGE_B;
    if (prv == lds) pprv = lds + (NS - 1) * STAGE_B;
    const uint32_t stage = ((wave & 2) ? prv : pprv) + (uint32_t)(wave & 1) * (uint32_t)(STAGE_B / 2);

    if (EPI == EPI_PARTIAL) {
      store_tile_partial<TM>(p, acc, em0, en0, bz, le, stage);
    } else if (EPI == EPI_TRANS) {
      load_bias<T, TM>(p, em0, en0, le, bias_regs);   // one round of latency, before any store is in flight
      store_tile_transcendental<T, TM>(p, acc, em0, en0, bz, le, stage, bias_regs);
    } else {
      if (EPI == EPI_BIAS) store_tile<T, TM, true, 0>(p, acc, em0, en0, bz, le, stage, bias_regs);
      else if (EPI == EPI_RELU) store_tile<T, TM, false, 1>(p, acc, em0, en0, bz, le, stage, bias_regs);
      else if (EPI == EPI_BIAS_RELU) store_tile<T, TM, true, 1>(p, acc, em0, en0, bz, le, stage, bias_regs);
      else if (EPI == EPI_CLIPPED) store_tile<T, TM, true, 2>(p, acc, em0, en0, bz, le, stage, bias_regs);
      else store_tile<T, TM, false, 0>(p, acc, em0, en0, bz, le, stage, bias_regs);
    }
    if (!has_next) break;

    // every wave has finished reading its staging area before any wave's loads overwrite it
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    v = vn;
    cur_tile = next_tile;
  }
}

#undef SRT_FENCE

template <typename T, bool A_KC, bool B_KC, int EPI, int NS, int TM = 8>
hipError_t launch_kernel(const GemmProblem& p, hipStream_t stream) {
  auto kernel = gemm_m16_kernel<T, A_KC, B_KC, EPI, NS, TM>;
  constexpr int tile_m = 32 * TM;
  constexpr int lds_bytes = NS * (tile_m * BK * 2 + REGION);
  static std::atomic<uint32_t> configured{0};
  if (hipError_t e = ensure_lds_limit(reinterpret_cast<const void*>(kernel), lds_bytes, configured); e != hipSuccess) return e;
  const long long tiles = (long long)((p.M + tile_m - 1) / tile_m) * ((p.N + BN - 1) / BN) * p.batch;
  const int grid = ring::persistent_grid(tiles);
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(NT), lds_bytes, stream, p);
  return launch_status(stream);
}

template <typename T, bool A_KC, bool B_KC, int NS = 5, int TM = 8>
hipError_t launch(const GemmProblem& p, hipStream_t stream) {
  const bool trans = p.activation == srtActivationSigmoid || p.activation == srtActivationTanh ||
                     p.activation == srtActivationElu;
  if (trans) return launch_kernel<T, A_KC, B_KC, EPI_TRANS, NS, TM>(p, stream);
  if (p.activation == srtActivationClippedRelu) return launch_kernel<T, A_KC, B_KC, EPI_CLIPPED, NS, TM>(p, stream);
  if (p.activation == srtActivationRelu) {
    if (p.bias) return launch_kernel<T, A_KC, B_KC, EPI_BIAS_RELU, NS, TM>(p, stream);
    return launch_kernel<T, A_KC, B_KC, EPI_RELU, NS, TM>(p, stream);
  }
  if (p.bias) return launch_kernel<T, A_KC, B_KC, EPI_BIAS, NS, TM>(p, stream);
  return launch_kernel<T, A_KC, B_KC, EPI_PLAIN, NS, TM>(p, stream);
}

// The split-K pass of `p` (whose C is the float workspace and whose batch counts the k ranges).
template <typename T, bool A_KC, bool B_KC, int NS = 5, int TM = 8>
hipError_t launch_partial(const GemmProblem& p, hipStream_t stream) {
  return launch_kernel<T, A_KC, B_KC, EPI_PARTIAL, NS, TM>(p, stream);
}

}  // namespace m16
}  // namespace srt
