// 256 x 256 bf16 / fp16 matmul tile kernel for gfx950 on v_mfma_f32_16x16x32 with operands staged
// 64 k deep: the kernel of gemm_mfma_m16.h (same wave tile, MFMA order, register use, epilogues and
// persistent tile walk) with the unit of staging doubled along k.
//
// Why.  A k-contiguous operand row holds 32 k in 64 bytes, half a cache line, so the 32-deep ring
// fetches every line of such an operand as two requests a stage apart.  With both operands stored that
// way (x . W^T) the loads, not the matrix pipe, set the pace: the 32-deep kernel reaches 1855 TFLOP/s on
// all-zero operands in that layout against 1985 in the others.  Its fragment reads, on the other hand,
// are the cheapest of all layouts -- a k-contiguous fragment is one ds_read_b128, and taking the fragment
// reads out of the loop gains 4 % there against 9-11 % where ds_read_b64_tr_b16 pairs are involved -- so
// under the power limit this is the layout with the most to gain from loads that move whole lines.
// A ring two stages deep is enough to hide the load latency (the 32-deep kernel measures the same with
// rings of 3, 4 and 5 stages), so the five 32 KiB slots are enough for 64-deep units.
//
// Unit of staging: one operand, 64 k deep, 32 KiB.  Units are numbered across the whole tile walk of a
// workgroup, A_0 B_0 A_1 B_1 ... (A_s / B_s: super-stage s), and unit u lives in slot u mod 5.
//   k-contiguous operand:  [256 rows][8 chunks of 16 B]; chunk c of row r at position c ^ ((r >> 1) & 7).
//                          A load instruction moves 8 rows x 128 B (whole lines); a fragment (16 rows x
//                          32 k) is one conflict-free ds_read_b128.
//   mn-contiguous operand: the 32-deep kernel's region [32 k][32 chunks] twice (k halves 16 KiB apart),
//                          its loads and its transposing reads.
// A super-stage is 128 MFMAs per wave in four phases of 32 -- (k half, A tiles): (0, 0-3) (0, 4-7) (1, 0-3)
// (1, 4-7) -- with the 32-deep kernel's register scheme: one register set per operand, tiles 4-7 read in
// the phase that multiplies tiles 0-3 of the same k half, tiles 0-3 of the next k half read during the
// phase before it.
//   phase 0, 1   the eight loads of A_{s+2} (its slot, that of B_{s-1}, fell free at the previous sync)
//   phase 2      --
//   sync         s_waitcnt vmcnt(8) lgkmcnt(0); s_barrier: every wave holds all of super-stage s in
//                registers (slots of A_s and B_s are free), A_{s+1} and B_{s+1} have landed for all
//   phase 3      the eight loads of B_{s+2} (into the slot of A_s), reads of super-stage s+1
// One barrier per 128 MFMAs.  Across tile boundaries the walk goes on: A'_0, B'_0 and A'_1 of the
// workgroup's next tile are requested while this tile's last super-stages are multiplied; the two slots
// vacated last are the epilogue's staging area and B'_1 is requested after it.
// Preconditions beyond the 32-deep kernel's: K a multiple of 64 and at least 256.
//
// A second form of the kernel (gemm_m16d_tail_kernel, "tail sharing") is for tile counts that leave some
// compute units without work in the last round: the tiles left over after the whole rounds are cut along k
// and all workgroups share them; see gemm_m16d_body.
#pragma once
#include "gemm_mfma_m16.h"

namespace srt {
namespace m16d {

using m16::EPI_BIAS;
using m16::EPI_BIAS_RELU;
using m16::EPI_CLIPPED;
using m16::EPI_PARTIAL;
using m16::EPI_PLAIN;
using m16::EPI_RELU;
using m16::EPI_TRANS;
using m16::EPI_SIGMOID;
using m16::EPI_TANH;
using m16::EPI_ELU;
using m16::mfma16;
using m16::mfma16_first;
using ring::BN;
using ring::f32x4_t;
using ring::NT;
using ring::OOB;
using ring::s16x4_t;
using ring::TileRef;
using ring::u32x2_t;
using ring::u32x4_t;

constexpr int DK = 64;               // k depth of a unit
constexpr int UNIT = 256 * DK * 2;   // bytes of a unit: 32 KiB
constexpr int UNITS = 5;             // slots: the whole LDS

#define SRT_FENCE() __builtin_amdgcn_sched_barrier(0)

// a < b ? t : f on the scalar unit.  Written out because the compiler, given one comparison with several
// selects behind it, keeps the (uniform) condition as a lane mask and selects on the vector unit -- and a
// value in a vector register cannot be the scalar offset of a buffer instruction.
__device__ __forceinline__ uint32_t select_lt(int a, int b, uint32_t t, uint32_t f) {
  uint32_t r;
  asm("s_cmp_lt_i32 %1, %2\n\ts_cselect_b32 %0, %3, %4" : "=s"(r) : "s"(a), "s"(b), "s"(t), "s"(f) : "scc");
  return r;
}

// ---- global -> LDS: eight loads per wave and unit ----------------------------------------------------
// A request is described by up to four scalar offsets so[j] (the unit's first byte in the operand plus
// j steps, or OOB); load i takes lane offset voff[vindex(i)], scalar offset so[sindex(i)] and lands
// landing(i) bytes into the wave's share of the slot.
// NL: loads per wave and unit -- 8 for a 256-wide unit, 4 for the 128-row k-contiguous A unit of the half tile.
template <bool KC, int NL = 8>
struct Loader {
  static_assert(NL == 8 || (KC && NL == 4), "an mn-contiguous unit is 256 wide");
  uint32_t voff[KC ? 2 : 4];
  static constexpr int SOFFS = KC ? NL / 2 : 2;
  static constexpr int vindex(int i) { return KC ? (i & 1) : (i & 3); }
  static constexpr int sindex(int i) { return KC ? (i >> 1) : (i >> 2); }
  static constexpr uint32_t landing(int i) { return KC ? (uint32_t)i * 1024u : (uint32_t)(i >> 2) * 16384u + (uint32_t)(i & 3) * 1024u; }
  static __device__ __forceinline__ uint32_t wave_share(int wave) { return (uint32_t)wave * (KC ? NL * 1024u : 4096u); }
  // bytes between so[j] and so[j + 1]: 16 rows (KC) or 32 k rows (MN)
  static __device__ __forceinline__ uint32_t step(long long ld) { return (uint32_t)((KC ? 16 : 32) * ld * 2); }

  // ld: elements between rows (KC) or between k (MN)
  __device__ __forceinline__ void init(int wave, int lane, long long ld) {
    if constexpr (KC) {
      // load i covers rows (NL wave + i) 8 .. + 7, 8 lanes per 128-byte row; (row >> 1) & 7 depends on the
      // lane and the parity of i only, so loads i and i + 2 differ by 16 rows in the scalar offset
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int row = (wave * NL + i) * 8 + (lane >> 3);
        const int chunk = (lane & 7) ^ ((row >> 1) & 7);
        voff[i] = (uint32_t)(((long long)row * ld + chunk * 8) * 2);
      }
    } else {
      // k half h = i >> 2 (32 k rows further: scalar offset); within it the 32-deep kernel's pattern
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int krow = (wave * 4 + i) * 2 + (lane >> 5);
        const int chunk = (lane & 31) ^ ((krow & 3) << 2) ^ (((krow >> 3) & 1) << 1);
        voff[i] = (uint32_t)(((long long)krow * ld + chunk * 8) * 2);
      }
    }
  }
};

// ---- LDS -> MFMA operands: 16 rows x 32 k of k half h ---------------------------------------------------
template <bool KC>
struct FragReader;
template <>
struct FragReader<true> {
  uint32_t off[2];   // per k half; tile t adds t * 2048
  __device__ __forceinline__ void init(int lane, int wave_row0) {
    const int g = lane >> 4, jn = lane & 15;
    const int f = (jn >> 1) & 7;   // (row >> 1) & 7 for rows wave_row0 + 16 t + jn
#pragma unroll
    for (int h = 0; h < 2; ++h) off[h] = (uint32_t)((wave_row0 + jn) * 128 + (((4 * h + g) ^ f) << 4));
  }
  template <int H>
  __device__ __forceinline__ u32x4_t read(uint32_t unit, int t) const {
    return *reinterpret_cast<const SRT_LDS u32x4_t*>(unit + off[H] + t * 2048);
  }
};
template <>
struct FragReader<false> {
  m16::FragReader<false> r;
  __device__ __forceinline__ void init(int lane, int wave_row0) { r.init(lane, wave_row0); }
  template <int H>
  __device__ __forceinline__ u32x4_t read(uint32_t unit, int t) const {
    return r.read(unit + H * 16384, t);
  }
};

// ---- the schedule's slots for a wave tile of TM x TN MFMA tiles (a phase is TM / 2 x TN MFMAs, u = TM / 2 j + i) ---------
// (TM, TN) = (8, 8) is the schedule as described above.  (8, 6) -- the 192-wide workgroup tile, 24 MFMAs per phase --,
// (4, 8) -- the 128 x 256 half tile, 16 MFMAs per phase, two A loads per phase -- and (8, 4) -- the 256 x 128 half tile,
// 16 MFMAs per phase -- keep the order of events and move them to earlier slots.  Every function gives, for MFMA u of a phase, the index of the thing that rides behind it, or -1.
template <int TM, int TN> constexpr int a_load_at(int u) {   // A load of the phase's share (phases 0, 1)
  if (TM == 4) return u == 12 ? 0 : u == 14 ? 1 : -1;
  if (TN == 4) return (u >= 8 && (u & 1) == 0) ? (u - 8) >> 1 : -1;
  return (u >= 4 * TN - 16 && (u & 3) == 0) ? (u - (4 * TN - 16)) >> 2 : -1;
}
template <int TM, int TN> constexpr int b_load_at(int u) {   // B load 0..7 (phase 3)
  if (TM == 4 || TN == 4) return (u & 1) == 0 ? u >> 1 : -1;
  return TN == 8 ? ((u & 3) == 0 ? u >> 2 : -1) : ((u % 3 == 0 && u < 24) ? u / 3 : -1);
}
// fragment reads of a phase that multiplies the first half of the A tiles (the rest of its own k half) ...
template <int TM, int TN> constexpr int own_b_read_at(int u) {   // B tiles 4 .. TN - 1
  if (TM == 4) return u < 4 ? 4 + u : -1;
  return (u < 8 && (u & 1) == 0 && 4 + (u >> 1) < TN) ? 4 + (u >> 1) : -1;
}
template <int TM, int TN> constexpr int own_a_read_at(int u) {   // A tiles TM / 2 .. TM - 1
  if (TM == 4) return (u == 4 || u == 5) ? 2 + (u - 4) : -1;
  if (TN == 4) return (u < 8 && (u & 1) == 1) ? 4 + (u >> 1) : -1;
  return (u >= 8 && u < 16 && (u & 1) == 0) ? 4 + ((u - 8) >> 1) : -1;
}
// ... and of one that multiplies the second half (tiles of the next k half: A 0 .. TM / 2 - 1, idle by now, and B 0-3,
// each right behind its last MFMA)
template <int TM> constexpr int next_a_read_at(int u) {
  if (TM == 4) return (u == 0 || u == 2) ? u >> 1 : -1;
  return (u < 16 && (u & 3) == 1) ? u >> 2 : -1;
}
template <int TM> constexpr int next_b_read_at(int u) {
  if (TM == 4) return (u < 8 && (u & 1) == 1) ? u >> 1 : -1;
  return (u < 16 && (u & 3) == 3) ? u >> 2 : -1;
}
// The slot of the (8, 8) schedule whose scalar bookkeeping happens behind MFMA u of phase PH
template <int TM, int TN, int PH> constexpr int event_at(int u) {
  if (TM == 4) {
    if (PH == 0) return (u >= 5 && u <= 11) ? 2 * (u - 5) + 1 : -1;             // 1, 3, .. 13 -> 5 .. 11 (loads at 12, 14)
    if (PH == 1) return u == 8 ? 10 : u == 10 ? 14 : -1;                         // 10, 14 -> 8, 10 (2 and 6: no third and fourth offset)
    if (PH == 2) return (u >= 7 && (u & 1) == 1) ? 17 + (u - 7) : -1;            // 17 .. 25 -> 7 .. 15
    return u == 9 ? 18 : u == 11 ? 22 : u == 13 ? 26 : -1;                       // 18, 22, 26 -> 9, 11, 13
  }
  if (TN == 8) return u;
  if (TN == 4) {
    if (PH == 0) return u < 7 ? 2 * u + 1 : -1;                                   // 1, 3, .. 13 -> 0 .. 6 (loads at 8, 10, 12, 14)
    if (PH == 1) return u;                                                        // 2, 6, 10, 14
    if (PH == 2) return (u >= 8 && u <= 12) ? 17 + 2 * (u - 8) : -1;              // 17 .. 25 -> 8 .. 12
    return u == 8 ? 18 : u == 10 ? 22 : u == 12 ? 26 : -1;                        // 18, 22, 26 -> 8, 10, 12 (behind a load each)
  }
  if (PH == 0) return u < 7 ? 2 * u + 1 : -1;                      // 1, 3, .. 13 -> 0 .. 6 (ahead of the loads from 8 on)
  if (PH == 1) return u;                                           // 2, 6, 10, 14
  if (PH == 2) return (u >= 15 && (u & 1) == 1) ? u + 2 : -1;      // 17 .. 25 -> 15 .. 23
  return u == 13 ? 18 : u == 17 ? 22 : u == 22 ? 26 : -1;          // 18, 22, 26 -> 13, 17, 22 (clear of the loads)
}

// The epilogue of the tail-sharing form: m16::store_tile (TM = 8) with switches that are uniform at run time,
// so that the kernel holds one copy of it and one place where the accumulators are read.  (With a copy per
// case the compiler moves all 256 accumulators out of their registers once, ahead of the branches, spilling
// what does not fit: every epilogue then took 23 us instead of 5.)
//   foreign   1 or 2: the tile's sum is spread over two or three workgroups; the accumulators of the other
//             one or two (f0, f1: what they published, see publish_accumulators) are added on the way out,
//             in the order of the parts along k whoever does the adding, streamed from memory four (one
//             foreign part) or two (two) rows of accumulator tiles ahead
// Partials are written and read with the agent-scope policy (cache policy operand 16: sc1): another
// workgroup, maybe on another XCD, reads or wrote them during this launch.
struct TailStore {
  __amdgpu_buffer_rsrc_t f0, f1;
  int foreign;
  bool own_last;   // foreign = 2: the sum is (f0 + f1) + own instead of (own + f0) + f1
};

// The accumulators to `mine` as they lie in the registers: [64 accumulator tiles][64 lanes][4] floats per
// wave.  Written out as instructions because they can take their data from the accumulator registers
// directly; through the compiler every value would first be copied to a vector register.
__device__ __forceinline__ void publish_accumulators(const f32x4_t (&acc)[8][8], u32x4_t mine, int lane) {
  const int lane16 = lane * 16;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
      asm volatile("buffer_store_dwordx4 %0, %1, %2, %3 offen sc1"
                   :: "a"(acc[i][j]), "v"(lane16), "s"(mine), "s"((i * 8 + j) * 1024) : "memory");
}

// FLIP: as m16::store_tile's -- the tile of row group i, column group j is acc[j][i], here and in what the other pieces
// published (every piece of a launch publishes its accumulators by their register index).
template <typename T, bool HAS_BIAS, int CLAMP, bool FLIP = false>
__device__ __forceinline__ void store_tile_tail(const GemmProblem& p, const f32x4_t (&acc)[8][8], int wave_m0, int wave_n0,
                                                int bz, int lane, uint32_t stage, const u32x2_t (&b)[8], const TailStore& t) {
  constexpr int AGENT = 16;
  using S = typename T::storage;
  const bool per_row = p.bias_per_row != 0;
  const float ceiling = p.coef;
  constexpr bool FIXUP = T::dtype == srtReal16BF;
  S* C = (S*)p.C + (long long)bz * p.scb;
  const long long c_last = (long long)(p.M - 1) * p.scm + p.N;
  const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc(C, 0, (int)(c_last * 2), 0x00020000);
  const int ldc2 = (int)(p.scm * 2);
  const int jn = lane & 15, g = lane >> 4;
  const int rd_chunk = lane & 15, rd_row = lane >> 4;
  const int n_rd = wave_n0 + 8 * rd_chunk;
  const bool n_rd_ok = n_rd < p.N;
  const int lane16 = lane * 16;
  const bool one = t.foreign >= 1, two = t.foreign == 2, last = t.own_last;

  // Four row slots of eight accumulator tiles each (128 registers).  One foreign part: row i lives in slot
  // i mod 4 and is requested four rows ahead; two: rows i of f0 and f1 live in slots 2 (i mod 2) and
  // 2 (i mod 2) + 1, two rows ahead.  Written and read under the same conditions.
  f32x4_t slots[4][8];
  auto fetch_row = [&](const __amdgpu_buffer_rsrc_t& from, int i, int slot) {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      slots[slot][j] = __builtin_bit_cast(f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(from, lane16, (FLIP ? j * 8 + i : i * 8 + j) * 1024, AGENT));
  };
  // what has to be requested once row `done` (-1: nothing yet) has been consumed
  auto fetch_after = [&](int done) {
    if (two) {
      const int i = done + 2;
      if (done < 0) {
        fetch_row(t.f0, 0, 0); fetch_row(t.f1, 0, 1); fetch_row(t.f0, 1, 2); fetch_row(t.f1, 1, 3);
      } else if (i < 8) {
        fetch_row(t.f0, i, 2 * (i % 2));
        fetch_row(t.f1, i, 2 * (i % 2) + 1);
      }
    } else if (one) {
      const int i = done + 4;
      if (done < 0) {
        fetch_row(t.f0, 0, 0); fetch_row(t.f0, 1, 1); fetch_row(t.f0, 2, 2); fetch_row(t.f0, 3, 3);
      } else if (i < 8) {
        fetch_row(t.f0, i, i % 4);
      }
    }
  };
  fetch_after(-1);

#pragma unroll
  for (int half = 0; half < 2; ++half) {
    bool nan = false;
#pragma unroll
    for (int ii = 0; ii < 4; ++ii) {
      const int i = 4 * half + ii;
      const int row = 16 * ii + jn;
      const uint32_t row_addr = stage + (uint32_t)row * 256u + (uint32_t)(g & 1) * 8u;
      SRT_FENCE();
      // the row's accumulators: one copy out of the accumulator registers, here, for every use
      float a[8][4];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const f32x4_t& tile = FLIP ? acc[j][i] : acc[i][j];
        a[j][0] = tile[0]; a[j][1] = tile[1]; a[j][2] = tile[2]; a[j][3] = tile[3];
        asm volatile("" : "+v"(a[j][0]), "+v"(a[j][1]), "+v"(a[j][2]), "+v"(a[j][3]));
      }
      if (two) {
        // (f0 + u) + w with (u, w) = (own, f1) or (f1, own)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const f32x4_t f0 = slots[2 * (i % 2)][j], f1 = slots[2 * (i % 2) + 1][j];
#pragma unroll
          for (int e = 0; e < 4; ++e) a[j][e] = (f0[e] + (last ? f1[e] : a[j][e])) + (last ? a[j][e] : f1[e]);
        }
      } else if (one) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const f32x4_t f0 = slots[i % 4][j];
#pragma unroll
          for (int e = 0; e < 4; ++e) a[j][e] += f0[e];
        }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float a0 = a[j][0], a1 = a[j][1], a2 = a[j][2], a3 = a[j][3];
        if (HAS_BIAS) {
          const float br = T::to_float((S)(b[i].x & 0xffffu));
          a0 += per_row ? br : T::to_float((S)(b[j].x & 0xffffu));
          a1 += per_row ? br : T::to_float((S)(b[j].x >> 16));
          a2 += per_row ? br : T::to_float((S)(b[j].y & 0xffffu));
          a3 += per_row ? br : T::to_float((S)(b[j].y >> 16));
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
        const int c = 2 * j + (g >> 1);
        *reinterpret_cast<SRT_LDS u32x2_t*>(row_addr + (uint32_t)((c ^ (row & 15)) << 4)) = w;
      }
      SRT_FENCE();
      fetch_after(i);   // the row's registers are free again
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
        const int m = wave_m0 + 64 * half + row;
        const uint32_t off = (n_rd_ok && m < p.M) ? (uint32_t)(m * ldc2 + n_rd * 2) : OOB;
        __builtin_amdgcn_raw_buffer_store_b128(v[q], rc, (int)off, 0, SRT_STORE_AUX);
      }
      SRT_FENCE();
    }
  }
}

// What the tail-sharing form of the kernel needs beyond the problem (see gemm_m16d_body, SK).
struct TailShare {
  float* partial;                // [left-over tile][part][wave][64 accumulator tiles][64 lanes][4] floats
  unsigned long long* flags;     // [left-over tile][part]: `epoch` once that piece's partial is complete
  unsigned int* stored;          // checking builds: [left-over tile] times the tile was stored (else unused)
  unsigned long long epoch;      // a value no earlier use of the memory has left there
  int parts;                     // pieces per left-over tile, 2 or 3
  int cut1, cut2;                // part k covers quads [cut(k), cut(k+1)): 0, cut1, cut2, quads per tile (cut2 = that for 2 parts)
  int groups;                    // workgroups that take the parts 1.. (a multiple of 8)
  int per_group;                 // pieces each of them takes at most
};
constexpr int TAIL_MAX_PARTS = 3;

// SK = false: workgroup w computes tiles w, w + G, ... whole.
// SK = true, the tail-sharing form, for a tile count that is not a multiple of G.  The tiles left over after
// the whole rounds (the last total mod G tile numbers) are cut along k, all at the same places (in quads: four
// super-stages), into 2 or 3 parts.  Workgroup i takes part 0 of left-over tile i; the other parts go to
// `groups` further workgroups, `per_group` pieces each, one after the other.  So every piece starts at the
// same k as its neighbours' and the workgroups of an XCD walk k together through a patch of tiles, as they do
// on whole tiles -- cut into runs of equal length instead, pieces start anywhere along k, no operand byte is
// shared in L2 and the walk is memory-bound (measured: a third slower than doing without).  (With workgroups
// dealt to the XCDs in turn all pieces of a tile are on one XCD; nothing relies on that.)  Each piece is a tile walk like any other -- its operand offsets start further along k
// and it has fewer super-stages -- so the k loop runs on across pieces as it does across tiles.  The piece
// of a tile that finishes last adds the others' accumulators to its own, in the order of the parts whoever
// it is (the bits do not depend on timing), and stores the tile; see the epilogue.  No workgroup ever waits
// for another, so the form makes no assumption about which workgroups are resident.  Every workgroup takes
// its pieces first and its whole tiles afterwards.
// FLIP: `p` describes the transposed product -- A is the caller's B^T, B the caller's A^T, M and N exchanged --
// while its result fields (C, its strides, the bias) are the caller's: the MFMAs take their operands in the
// other order, so that every accumulator tile lies in the registers as the epilogue expects it, and the epilogue
// addresses the tile block transposed.  For a k-contiguous A against an n-contiguous B this makes the operand
// with the transposing LDS reads the one whose fragments are read four tiles per phase (1512 -> 1540 TFLOP/s at
// 8192^3: the kernel runs 2 % faster whenever its B is k-contiguous, whatever A is).
// TN: column tiles per wave.  8: the 256 x 256 tile.  6: a workgroup tile of 256 x 192 MFMA footprint (waves of 128 x 96)
// whose valid width p.tile_n <= 192 is a multiple of 8 -- tiles lie p.tile_n columns apart and columns beyond that
// width are computed and not stored.  It fills a last round of the persistent grid that whole tiles would leave three
// quarters full or less (see gemm_m16d_split_kernel).  B is staged as for the wide tile (a 256-wide unit).
// 4: the 256 x 128 half tile (waves of 128 x 64; p.tile_n <= 128), which gives an A that is not k-contiguous -- and so has
// no 128 x 256 half tile -- twice the workgroups on a partly filled device.  The B unit stays 256 wide in LDS; of a
// k-contiguous B only the first 128 rows are requested (the loads of waves 2 and 3 aim out of range), an n-contiguous
// B's k rows are fetched whole (the tile's neighbour's columns ride along).
// TM: row tiles per wave.  8: 256 rows per workgroup tile.  4: the 128 x 256 half tile (waves of 64 x 128) for problems that
// leave compute units idle with whole tiles; its A unit is 128 rows of a k-contiguous A (in a slot of the same size).
template <typename T, bool A_KC, bool B_KC, int EPI, bool SK, bool FLIP = false, int TN = 8, int TM = 8>
__device__ __forceinline__ void gemm_m16d_body(const GemmProblem& p, const TailShare& ts) {
  static_assert(EPI != EPI_TRANS, "sigmoid / tanh / elu have epilogue kinds of their own here");
  static_assert(!FLIP || EPI != EPI_PARTIAL, "flipped: the store_tile epilogues only");
  static_assert(TN == 8 || ((TN == 6 || TN == 4) && !SK && !FLIP && EPI != EPI_PARTIAL), "the narrow tiles: plain form, store_tile epilogues");
  static_assert(TM == 8 || (TM == 4 && TN == 8 && A_KC && !SK && !FLIP), "the half tile: k-contiguous A, plain form");
  constexpr int HALF = TM / 2;        // A tiles per phase
  constexpr int TILE_M = 32 * TM;     // rows of a workgroup tile
  constexpr int NLA = TM;             // A loads per wave and unit
  using LoaderA = Loader<A_KC, NLA>;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[];
  const uint32_t lds = (uint32_t)(uintptr_t)(SRT_LDS unsigned char*)lds_raw;
  const uint32_t lds_end = lds + UNITS * UNIT;

  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  auto lane_id = []() {
    uint32_t zero = 0;
    asm volatile("" : "+s"(zero));   // opaque: keeps the two instructions where they are written
    return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, zero));
  };
  const int wm0 = (wave >> 1) * (16 * TM), wn0 = (wave & 1) * (16 * TN);

  const int tile_w = TN == 8 ? BN : p.tile_n;   // columns between neighbouring tiles
  const int tiles_m = (p.M + TILE_M - 1) / TILE_M, tiles_n = (p.N + tile_w - 1) / tile_w;
  const int total = tiles_m * tiles_n * p.batch;
  const int grid = (int)gridDim.x;
  int v = (int)blockIdx.x;

  const long long lda = A_KC ? p.sam : p.sak;
  const long long ldb = B_KC ? p.sbn : p.sbk;
  const long long a_view = A_KC ? (long long)(p.M - 1) * lda + p.K : (long long)(p.K - 1) * lda + p.M;
  const long long b_view = B_KC ? (long long)(p.N - 1) * ldb + p.K : (long long)(p.K - 1) * ldb + p.N;
  const u32x4_t ra = ring::make_rsrc(p.A, (uint32_t)(((long long)(p.batch - 1) * p.sab + a_view) * 2));
  const u32x4_t rb = ring::make_rsrc(p.B, (uint32_t)(((long long)(p.batch - 1) * p.sbb + b_view) * 2));
  // tile number -> position and operand offsets (the narrow tile's columns lie tile_w apart)
  auto locate = [&](int tile) {
    TileRef t = m16::locate_tile<A_KC, B_KC, TILE_M>(p, tile, tiles_m, tiles_n);
    if constexpr (TN != 8) {
      t.n0 = (t.n0 / BN) * tile_w;
      t.offb = (uint32_t)(((long long)t.bz * p.sbb + (B_KC ? (long long)t.n0 * ldb : (long long)t.n0)) * 2);
    }
    return t;
  };
  const uint32_t kstep_a = A_KC ? (uint32_t)(DK * 2) : (uint32_t)(DK * lda * 2);   // bytes per super-stage
  const uint32_t kstep_b = B_KC ? (uint32_t)(DK * 2) : (uint32_t)(DK * ldb * 2);
  const uint32_t lstep_a = LoaderA::step(lda), lstep_b = Loader<B_KC>::step(ldb);
  const int S_full = p.K / DK;   // super-stages per tile (the host admits whole ones only, at least four)

  // per-XCD start of the k walk for an A stored k x m (see gemm_ring_kernel)
  constexpr bool rotate = !A_KC;
  const int rot = rotate && !SK ? (int)(((unsigned)(blockIdx.x & 7) * (unsigned)S_full) / 8u) : 0;
  auto stage_of = [&](int r) {   // r = 0, 1, 2 only; a piece has at least four super-stages
    if constexpr (SK) return r;
    int e = r + rot;
    e = e >= S_full ? e - S_full : e;
    e = e >= S_full ? e - S_full : e;
    return e;
  };
  auto wrap = [&](uint32_t a) { return a >= lds_end ? a - UNITS * UNIT : a; };

  // ---- the walk: pieces of work, each a tile or (SK) some quads of one ----
  struct Piece {
    TileRef t;   // offa / offb already advanced to the piece's first super-stage
    int n;       // super-stages
    int tile;    // SK: index among the left-over tiles when the piece is a part of one, else -1
    int part;
  };
  // an explicit move to the scalar unit (what feeds a scalar operand of an instruction written out below
  // must be in a scalar register, and the compiler keeps some uniform values in vector ones)
  // The compiler does not see inside the statement, so the wait states this instruction needs on gfx950 are
  // written out: one after a vector write of the register it reads (the copy into it may be the
  // instruction just before -- without the s_nop the read returned the register's previous content), and
  // those between a vector write of a scalar register and its use by a vector (2) or memory (5) instruction.
  auto scalar = [](int x) {
    int r;
    asm volatile("s_nop 0\n\tv_readfirstlane_b32 %0, %1\n\ts_nop 4" : "=s"(r) : "v"(x));
    return r;
  };
  const int rounds = total / grid;
  const int left = total - rounds * grid;       // SK: the last `left` tile numbers are the shared ones
  const int left8 = (left + 7) & ~7;
  const int Q = S_full >> 2;                    // quads per tile
  auto cut = [&](int k) { return k == 0 ? 0 : k == 1 ? ts.cut1 : k == 2 ? ts.cut2 : Q; };
  int taken = 0;   // SK: pieces taken so far (or tried)
  int round = 0;   // SK: whole tiles taken so far
  const int me = (int)blockIdx.x;
  auto take = [&](Piece& w) {   // SK only; false when the workgroup has nothing left
    int tile = -1, part = 0;
    if (me < left) {
      if (taken == 0) tile = me;
      taken = 1;
    } else if (me >= left8 && me - left8 < ts.groups) {
      while (tile < 0 && taken < ts.per_group) {
        const int e = me - left8 + taken * ts.groups;
        ++taken;
        if (e < (ts.parts - 1) * left8 && e % left8 < left) {
          tile = e % left8;
          part = 1 + e / left8;
        }
      }
    }
    if (tile >= 0) {
      const int s0 = cut(part) * 4;
      w.t = m16::locate_tile<A_KC, B_KC, 256>(p, rounds * grid + tile, tiles_m, tiles_n);
      w.t.offa += (uint32_t)s0 * kstep_a;
      w.t.offb += (uint32_t)s0 * kstep_b;
      w.n = (cut(part + 1) - cut(part)) * 4;
      w.tile = tile;
      w.part = part;
      return true;
    }
    if (round < rounds) {
      w.t = m16::locate_tile<A_KC, B_KC, 256>(p, me + round * grid, tiles_m, tiles_n);
      w.n = S_full;
      w.tile = -1;
      w.part = 0;
      ++round;
      return true;
    }
    return false;
  };
  auto uniform = [&](Piece& w) {
    w.t.offa = (uint32_t)scalar((int)w.t.offa);
    w.t.offb = (uint32_t)scalar((int)w.t.offb);
    w.n = scalar(w.n);
  };

  TileRef cur_tile;
  Piece cur_piece, next_piece;
  if constexpr (SK) {
    if (!take(cur_piece)) return;
    uniform(cur_piece);
    cur_tile = cur_piece.t;
  } else {
    if (v >= total) return;   // (a walk with fewer tiles than workgroups: the split kernel's)
    cur_tile = locate(v);
  }

  // the eight loads of one unit, outside the main loop (first fill, and B_1 after an epilogue)
  auto issue_a = [&](const LoaderA& l, uint32_t slot, uint32_t base) {
#pragma unroll
    for (int i = 0; i < NLA; ++i)
      ring::load_to_lds(ra, slot + LoaderA::wave_share(wave) + LoaderA::landing(i),
                        l.voff[LoaderA::vindex(i)], base + (uint32_t)LoaderA::sindex(i) * lstep_a);
  };
  auto issue_b = [&](const Loader<B_KC>& l, uint32_t slot, uint32_t base) {
    if constexpr (TN == 4 && B_KC) base = select_lt(wave, 2, base, OOB);   // rows 128-255 of the unit are not needed
#pragma unroll
    for (int i = 0; i < 8; ++i)
      ring::load_to_lds(rb, slot + Loader<B_KC>::wave_share(wave) + Loader<B_KC>::landing(i),
                        l.voff[Loader<B_KC>::vindex(i)], base + (uint32_t)Loader<B_KC>::sindex(i) * lstep_b);
  };

  uint32_t x = lds;   // slot of A_s; B_s follows it, then A_{s+1}, B_{s+1}, A_{s+2} (B_{s+2} goes where A_s is)

  bool first_tile = true;
  for (;;) {
    // per-lane addressing state, derived per tile and scoped to it (see gemm_ring_kernel)
    LoaderA la;
    Loader<B_KC> lb;
    FragReader<A_KC> fa;
    FragReader<B_KC> fb;
    const int lane = lane_id();
    la.init(wave, lane, lda);
    lb.init(wave, lane, ldb);
    fa.init(lane, wm0);
    fb.init(lane, wn0);
    uint32_t xb = wrap(x + UNIT), xa1 = wrap(x + 2 * UNIT), xb1 = wrap(x + 3 * UNIT);
    if (first_tile) {
      issue_a(la, x, cur_tile.offa + (uint32_t)stage_of(0) * kstep_a);
      issue_b(lb, xb, cur_tile.offb + (uint32_t)stage_of(0) * kstep_b);
      issue_a(la, xa1, cur_tile.offa + (uint32_t)stage_of(1) * kstep_a);
      issue_b(lb, xb1, cur_tile.offb + (uint32_t)stage_of(1) * kstep_b);
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" : : "i"(NLA + 8) : "memory");
    } else {
      issue_b(lb, xb1, cur_tile.offb + (uint32_t)stage_of(1) * kstep_b);
    }
    first_tile = false;
    SRT_FENCE();

    int vn = 0, S = S_full;
    bool has_next;
    TileRef next_tile;
    if constexpr (SK) {
      S = cur_piece.n;
      has_next = take(next_piece);
      if (!has_next) next_piece = cur_piece;
      uniform(next_piece);
      next_tile = next_piece.t;
      vn = scalar(has_next ? 0 : 1);   // vn < 1 below: there is a next piece
    } else {
      vn = v + grid;
      has_next = vn < total;
      next_tile = locate((int)select_lt(vn, total, (uint32_t)vn, (uint32_t)v));
    }
    const int vn_bound = SK ? 1 : total;
    // A requests below limit_a are real (A'_0 and A'_1 of the next tile); of B only B'_0: B'_1 would land in
    // the staging area
    const int limit_a = (int)select_lt(vn, vn_bound, (uint32_t)(S + 2), (uint32_t)S);
    const int limit_b = (int)select_lt(vn, vn_bound, (uint32_t)(S + 1), (uint32_t)S);

    f32x4_t acc[TM][TN];   // defined by the MFMAs of the tile's first super-stage
    u32x4_t af[TM], bf[TN];
#pragma unroll
    for (int t = 0; t < 4; ++t) bf[t] = fb.template read<0>(xb, t);
#pragma unroll
    for (int t = 0; t < HALF; ++t) af[t] = fa.template read<0>(x, t);

    int e_req = stage_of(2);   // k index of request s + 2
    uint32_t ea_off = (uint32_t)e_req * kstep_a, eb_off = (uint32_t)e_req * kstep_b;

    auto set_target = [](auto imm_tag, uint32_t base) __attribute__((always_inline)) {
      ring::set_lds_target<decltype(imm_tag)::value>(base);
    };

    // One phase: 32 MFMAs, B tile by B tile (u = 4 j + i), on A tiles 4 AH .. 4 AH + 3.
    //   OWN  (phases 0, 2): reads B tiles 4-7 and A tiles 4-7 of k half H from (ua, ub)
    //   !OWN (phases 1, 3): reads A tiles 0-3 and B tiles 0-3 of k half H from (ua, ub) -- the next k half
    //   LOADS 0: none; 1: A loads 0-3; 2: A loads 4-7 (second half of the phase); 3: B loads 0-7 (whole phase)
    // `so`: the request's scalar offsets; `target`: its slot plus the wave's share.  `ev(u)`: scalar bookkeeping.
    auto phase = [&](auto ah_tag, auto first_tag, auto own_tag, auto h_tag, auto loads_tag, uint32_t ua, uint32_t ub,
                     const uint32_t& target, const uint32_t& so0, const uint32_t& so1, const uint32_t& so2,
                     const uint32_t& so3, auto&& ev) __attribute__((always_inline)) {
      constexpr int AH = decltype(ah_tag)::value;
      constexpr bool FIRST = decltype(first_tag)::value;
      constexpr bool OWN = decltype(own_tag)::value;
      constexpr int H = decltype(h_tag)::value;
      constexpr int LOADS = decltype(loads_tag)::value;
      constexpr int PH = LOADS == 1 ? 0 : LOADS == 2 ? 1 : LOADS == 0 ? 2 : 3;   // the phase's number
#pragma unroll
      for (int j = 0; j < TN; ++j) {
#pragma unroll
        for (int i = 0; i < HALF; ++i) {
          const int u = HALF * j + i;
          // which load, if any, rides on this MFMA
          const int ld = LOADS == 3 ? b_load_at<TM, TN>(u)
                       : (LOADS == 1 || LOADS == 2) ? (a_load_at<TM, TN>(u) >= 0 ? a_load_at<TM, TN>(u) + (LOADS == 2 ? NLA / 2 : 0) : -1)
                       : -1;
          if (ld >= 0) {
            if (LOADS == 3) {
              constexpr uint32_t imm[8] = {Loader<B_KC>::landing(0), Loader<B_KC>::landing(1), Loader<B_KC>::landing(2),
                                           Loader<B_KC>::landing(3), Loader<B_KC>::landing(4), Loader<B_KC>::landing(5),
                                           Loader<B_KC>::landing(6), Loader<B_KC>::landing(7)};
              if (ld == 0) set_target(std::integral_constant<uint32_t, imm[0]>{}, target);
              if (ld == 1) set_target(std::integral_constant<uint32_t, imm[1]>{}, target);
              if (ld == 2) set_target(std::integral_constant<uint32_t, imm[2]>{}, target);
              if (ld == 3) set_target(std::integral_constant<uint32_t, imm[3]>{}, target);
              if (ld == 4) set_target(std::integral_constant<uint32_t, imm[4]>{}, target);
              if (ld == 5) set_target(std::integral_constant<uint32_t, imm[5]>{}, target);
              if (ld == 6) set_target(std::integral_constant<uint32_t, imm[6]>{}, target);
              if (ld == 7) set_target(std::integral_constant<uint32_t, imm[7]>{}, target);
            } else {
              constexpr uint32_t imm[8] = {LoaderA::landing(0), LoaderA::landing(1), LoaderA::landing(2),
                                           LoaderA::landing(3), LoaderA::landing(4), LoaderA::landing(5),
                                           LoaderA::landing(6), LoaderA::landing(7)};
              if (ld == 0) set_target(std::integral_constant<uint32_t, imm[0]>{}, target);
              if (ld == 1) set_target(std::integral_constant<uint32_t, imm[1]>{}, target);
              if (ld == 2) set_target(std::integral_constant<uint32_t, imm[2]>{}, target);
              if (ld == 3) set_target(std::integral_constant<uint32_t, imm[3]>{}, target);
              if (ld == 4) set_target(std::integral_constant<uint32_t, imm[4]>{}, target);
              if (ld == 5) set_target(std::integral_constant<uint32_t, imm[5]>{}, target);
              if (ld == 6) set_target(std::integral_constant<uint32_t, imm[6]>{}, target);
              if (ld == 7) set_target(std::integral_constant<uint32_t, imm[7]>{}, target);
            }
            SRT_FENCE();
          }
          if constexpr (FLIP) {   // A fragment first: the tile comes out as the transposed product's
            if constexpr (FIRST) mfma16_first<T>(acc[HALF * AH + i][j], af[HALF * AH + i], bf[j]);
            else mfma16<T>(acc[HALF * AH + i][j], af[HALF * AH + i], bf[j]);
          } else {
            if constexpr (FIRST) mfma16_first<T>(acc[HALF * AH + i][j], bf[j], af[HALF * AH + i]);
            else mfma16<T>(acc[HALF * AH + i][j], bf[j], af[HALF * AH + i]);
          }
          if (ld >= 0) {
            SRT_FENCE();
            const int si = LOADS == 3 ? Loader<B_KC>::sindex(ld) : LoaderA::sindex(ld);
            const uint32_t so = si == 0 ? so0 : si == 1 ? so1 : si == 2 ? so2 : so3;
            if (LOADS == 3) ring::load_to_lds_at_m0(rb, lb.voff[Loader<B_KC>::vindex(ld)], so);
            else ring::load_to_lds_at_m0(ra, la.voff[LoaderA::vindex(ld)], so);
          }
          if (OWN) {
            if (own_b_read_at<TM, TN>(u) >= 0) bf[own_b_read_at<TM, TN>(u)] = fb.template read<H>(ub, own_b_read_at<TM, TN>(u));
            if (own_a_read_at<TM, TN>(u) >= 0) af[own_a_read_at<TM, TN>(u)] = fa.template read<H>(ua, own_a_read_at<TM, TN>(u));
          } else {
            if (next_a_read_at<TM>(u) >= 0) af[next_a_read_at<TM>(u)] = fa.template read<H>(ua, next_a_read_at<TM>(u));
            if (next_b_read_at<TM>(u) >= 0) bf[next_b_read_at<TM>(u)] = fb.template read<H>(ub, next_b_read_at<TM>(u));
          }
          ev(event_at<TM, TN, PH>(u));
          SRT_FENCE();
        }
      }
    };

    using C0 = std::integral_constant<int, 0>;
    using C1 = std::integral_constant<int, 1>;
    using C2 = std::integral_constant<int, 2>;
    using C3 = std::integral_constant<int, 3>;
    auto super_stage = [&](auto first_tag, int s) __attribute__((always_inline)) {
      const int r = s + 2;   // index of the units requested in this super-stage
      uint32_t xa2 = 0, sel = 0, soa = 0, sob = 0, ta = 0, tb = 0;
      uint32_t so_a0 = OOB, so_a1 = OOB, so_a2 = OOB, so_a3 = OOB, so_b0 = OOB, so_b1 = OOB, so_b2 = OOB, so_b3 = OOB;
      // ---- phase 0: k half 0, A tiles 0-3; loads 0-3 of A_{s+2} ----
      phase(C0{}, first_tag, std::true_type{}, C0{}, C1{}, x, xb, ta, so_a0, so_a1, so_a2, so_a3, [&](int u) __attribute__((always_inline)) {
        if (u == 1) xa2 = xa1 + 2 * UNIT;
        if (u == 3) xa2 = select_lt((int)xa2, (int)lds_end, xa2, xa2 - UNITS * UNIT);
        if (u == 5) sel = select_lt(r, S, cur_tile.offa, next_tile.offa);
        if (u == 7) soa = select_lt(r, limit_a, sel + ea_off, OOB);
        if (u == 9) ta = xa2 + LoaderA::wave_share(wave);
        if (u == 11) so_a0 = soa;
        if (u == 13) so_a1 = select_lt(r, limit_a, soa + lstep_a, OOB);
      });
      // ---- phase 1: k half 0, A tiles 4-7; loads 4-7 of A_{s+2}; reads of k half 1 ----
      phase(C1{}, first_tag, std::false_type{}, C1{}, C2{}, x, xb, ta, so_a0, so_a1, so_a2, so_a3, [&](int u) __attribute__((always_inline)) {
        if (LoaderA::SOFFS == 4) {
          if (u == 2) so_a2 = select_lt(r, limit_a, soa + 2 * lstep_a, OOB);
          if (u == 6) so_a3 = select_lt(r, limit_a, soa + 3 * lstep_a, OOB);
        }
        if (u == 10) sel = select_lt(r, S, cur_tile.offb, next_tile.offb);
        if (u == 14) {
          sob = select_lt(r, limit_b, sel + eb_off, OOB);
          if constexpr (TN == 4 && B_KC) sob = select_lt(wave, 2, sob, OOB);   // rows 128-255 of the unit are not needed
        }
      });
      // ---- phase 2: k half 1, A tiles 0-3 ----
      phase(C0{}, std::false_type{}, std::true_type{}, C1{}, C0{}, x, xb, ta, so_a0, so_a1, so_a2, so_a3, [&](int u) __attribute__((always_inline)) {
        if (u == 17) so_b0 = sob;
        if (u == 19) so_b1 = select_lt(r, limit_b, sob + lstep_b, OOB);
        if (Loader<B_KC>::SOFFS == 4) {
          if (u == 21) so_b2 = select_lt(r, limit_b, sob + 2 * lstep_b, OOB);
          if (u == 23) so_b3 = select_lt(r, limit_b, sob + 3 * lstep_b, OOB);
        }
        if (u == 25) tb = x + Loader<B_KC>::wave_share(wave);
      });
      // ---- sync: all of super-stage s is in registers, A_{s+1} and B_{s+1} have landed ----
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" : : "i"(NLA) : "memory");
      SRT_FENCE();
      // ---- phase 3: k half 1, A tiles 4-7; the loads of B_{s+2}; reads of super-stage s + 1 ----
      phase(C1{}, std::false_type{}, std::false_type{}, C0{}, C3{}, xa1, xb1, tb, so_b0, so_b1, so_b2, so_b3, [&](int u) __attribute__((always_inline)) {
        // the next request's k index: one further, or back to 0 past the tile's last super-stage
        if (u == 18) ea_off = select_lt(e_req + 1, S, ea_off + kstep_a, 0u);
        if (u == 22) eb_off = select_lt(e_req + 1, S, eb_off + kstep_b, 0u);
        if (u == 26) e_req = (int)select_lt(e_req + 1, S, (uint32_t)(e_req + 1), 0u);
      });
      // the slots move on by one super-stage: B_{s+3} will go where B_s... A_{s+1} becomes A_s
      const uint32_t old_x = x;
      x = xa1;
      xb = xb1;
      xa1 = xa2;
      xb1 = old_x;
    };
    super_stage(std::true_type{}, 0);
    {
      int s = 1;   // S >= 4: no guard in front of the loop
      do super_stage(std::false_type{}, s); while (++s < S);
    }

    // Every load in flight must have landed, in every wave, before the slots vacated last become the
    // staging area.  The s_nops are the wait states between the last MFMAs and the first reads of their
    // accumulators by other instructions.
    // (flipped: the result's rows are this problem's columns)
    const int em0 = FLIP ? cur_tile.n0 + wn0 : cur_tile.m0 + wm0, en0 = FLIP ? cur_tile.m0 + wm0 : cur_tile.n0 + wn0;
    const int bz = cur_tile.bz;
    GemmProblem pe = p;   // the problem as the epilogue sees it
    if (FLIP) { pe.M = p.N; pe.N = p.M; }
    const int le = lane_id();
    constexpr bool LINEAR_BIAS = EPI == EPI_BIAS || EPI == EPI_BIAS_RELU || EPI == EPI_CLIPPED || EPI == EPI_SIGMOID ||
                                 EPI == EPI_TANH || EPI == EPI_ELU;
    u32x2_t bias_regs[8];
    if (LINEAR_BIAS) m16::load_bias<T, TM>(pe, em0, en0, le, bias_regs);   // lands during the wait below
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier\n\ts_nop 7\n\ts_nop 7" ::: "memory");
    if (LINEAR_BIAS || SK) m16::pin_all<TM>(acc);
    const int n_end = cur_tile.n0 + tile_w;   // (the narrow tile: its valid columns end here)
    // staging: the slots of A_{S-1} (waves 0, 1) and B_{S-1} (waves 2, 3), half a slot each; x is A_S's by now
    uint32_t sa = x < lds + 2 * UNIT ? x + 3 * UNIT : x - 2 * UNIT;
    uint32_t sb = x < lds + UNIT ? x + 4 * UNIT : x - UNIT;
    const uint32_t stage = ((wave & 2) ? sb : sa) + (uint32_t)(wave & 1) * (uint32_t)(UNIT / 2);

    if constexpr (SK) {
      // One copy of the epilogue (store_tile_tail), run once or twice.
      // A whole tile: once, plain.  A part of a tile: whichever piece of the tile finds the flags of all
      // the others raised adds up the partials in the order of the parts -- its own straight from the
      // registers -- and stores the tile; a piece that does not leaves its accumulators in `partial`
      // (first run), raises its flag and looks again: of two pieces that finish together at least one
      // then sees the other, and if both do, both store the same bits (second run).  Nobody waits.
      // Coherence between workgroups is per access, not per cache: partials and flags are written and read
      // with the agent-scope policy (sc1: stores write through, loads do not trust a cached copy), and
      // s_waitcnt vmcnt(0) -- the stores have been acknowledged -- orders partials before the flag and the
      // flag before the second look.  (Agent-scope fences would write back and invalidate whole L2s, once
      // per workgroup: measured at 100 us per launch.)
      const bool part_of_tile = cur_piece.tile >= 0;
      const int place0 = part_of_tile ? cur_piece.tile * ts.parts : 0, mine = cur_piece.part;
      auto others_done = [&]() {
        bool ok = true;
        for (int k = 0; k < ts.parts; ++k)
          if (k != mine)
            ok &= __hip_atomic_load(ts.flags + place0 + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == ts.epoch;
        return ok;
      };
      // one thread decides for the workgroup; the verdict travels through the first word of the staging area
      SRT_LDS int* verdict = reinterpret_cast<SRT_LDS int*>(sa);
      auto agree = [&](auto&& decide) {
        if (threadIdx.x == 0) *verdict = decide() ? 1 : 0;
        __syncthreads();
        const int v = __builtin_amdgcn_readfirstlane(*verdict);
        __syncthreads();
        return v != 0;
      };
      auto partial_of = [&](int part) {   // (a whole tile has no partials: an empty descriptor on the workspace's start)
        float* base = ts.partial + (part_of_tile ? ((size_t)((place0 + part) * 4 + wave) * 64) * 256 : 0);
        return __builtin_amdgcn_make_buffer_rsrc(base, 0, part_of_tile ? 65536 : 0, 0x00020000);
      };
      TailStore how;
      how.foreign = 0;
      how.own_last = false;
      // the other parts in order: f0, then f1 if there are three
      const int o0 = mine == 0 ? 1 : 0;
      const int o1 = ts.parts == 3 ? (mine == 2 ? 1 : 2) : o0;
      how.f0 = partial_of(o0);
      how.f1 = partial_of(o1);
      // part 0 is expected to end last (see tail_plan) and looks first; the others publish first
      constexpr bool HAS_BIAS = EPI == EPI_BIAS || EPI == EPI_BIAS_RELU || EPI == EPI_CLIPPED;
      constexpr int CLAMP = EPI == EPI_CLIPPED ? 2 : (EPI == EPI_RELU || EPI == EPI_BIAS_RELU) ? 1 : 0;
      bool finish = true;
      if (part_of_tile) finish = mine == 0 && agree(others_done);
      for (;;) {
        if (finish) {
          if (part_of_tile) {
            how.foreign = ts.parts - 1;
            how.own_last = mine == 2;
          }
          m16::pin_all<TM>(acc);   // (nothing read from the accumulators moves out of the loop)
          store_tile_tail<T, HAS_BIAS, CLAMP, FLIP>(pe, acc, em0, en0, bz, lane_id(), stage, bias_regs, how);
#ifdef SRT_DEBUG_LAUNCH
          // checking builds count the stores of every shared tile; the host reads the counts after the launch
          if (part_of_tile && threadIdx.x == 0) atomicAdd(ts.stored + cur_piece.tile, 1u);
#endif
          break;
        }
        publish_accumulators(acc, ring::make_rsrc(ts.partial + ((size_t)((place0 + mine) * 4 + wave) * 64) * 256, 65536), lane_id());
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        finish = agree([&]() {
          __hip_atomic_store(ts.flags + place0 + mine, ts.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          return others_done();
        });
        if (!finish) break;
      }
    } else if constexpr (EPI == EPI_PARTIAL) {
      m16::store_tile_partial<TM>(p, acc, em0, en0, bz, le, stage);
    } else {
      if (EPI == EPI_BIAS) m16::store_tile<T, TM, true, 0, FLIP>(pe, acc, em0, en0, bz, le, stage, bias_regs, n_end);
      else if (EPI == EPI_RELU) m16::store_tile<T, TM, false, 1, FLIP>(pe, acc, em0, en0, bz, le, stage, bias_regs, n_end);
      else if (EPI == EPI_BIAS_RELU) m16::store_tile<T, TM, true, 1, FLIP>(pe, acc, em0, en0, bz, le, stage, bias_regs, n_end);
      else if (EPI == EPI_CLIPPED) m16::store_tile<T, TM, true, 2, FLIP>(pe, acc, em0, en0, bz, le, stage, bias_regs, n_end);
      else if (EPI == EPI_SIGMOID) m16::store_tile<T, TM, true, 3, FLIP>(pe, acc, em0, en0, bz, le, stage, bias_regs, n_end);
      else if (EPI == EPI_TANH) m16::store_tile<T, TM, true, 4, FLIP>(pe, acc, em0, en0, bz, le, stage, bias_regs, n_end);
      else if (EPI == EPI_ELU) m16::store_tile<T, TM, true, 5, FLIP>(pe, acc, em0, en0, bz, le, stage, bias_regs, n_end);
      else m16::store_tile<T, TM, false, 0, FLIP>(pe, acc, em0, en0, bz, le, stage, bias_regs, n_end);
    }
    if (!has_next) break;

    // every wave has finished reading its staging area before any wave's loads overwrite it
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if constexpr (SK) cur_piece = next_piece;
    else v = vn;
    cur_tile = next_tile;
  }
}

template <typename T, bool A_KC, bool B_KC, int EPI, bool FLIP = false>
__global__ __launch_bounds__(NT) void gemm_m16d_kernel(GemmProblem p) {
  gemm_m16d_body<T, A_KC, B_KC, EPI, false, FLIP>(p, TailShare{});
}

template <typename T, bool A_KC, bool B_KC, int EPI, bool FLIP = false>
__global__ __launch_bounds__(NT) void gemm_m16d_tail_kernel(GemmProblem p, TailShare ts) {
  gemm_m16d_body<T, A_KC, B_KC, EPI, true, FLIP>(p, ts);
}

// The 128 x 256 half tile (k-contiguous A), for problems that leave compute units idle with whole tiles.
template <typename T, bool B_KC, int EPI>
__global__ __launch_bounds__(NT) void gemm_m16d_half_kernel(GemmProblem p) {
  gemm_m16d_body<T, true, B_KC, EPI, false, false, 8, 4>(p, TailShare{});
}

// The 256 x 128 half tile, for an A that is not k-contiguous.
template <typename T, bool B_KC, int EPI>
__global__ __launch_bounds__(NT) void gemm_m16d_narrow_kernel(GemmProblem p) {
  gemm_m16d_body<T, false, B_KC, EPI, false, false, 4, 8>(p, TailShare{});
}

// Two tile walks in one launch, for a tile count that leaves the last round of the persistent grid between half
// and three quarters full (688 tiles on 256 units: 2.69 rounds, 3 paid).  The columns are cut in two: `wide` covers
// the first columns in whole 256 x 256 tiles that fill whole rounds (it is the problem as the plain kernel would get
// it, flipped where that one flips), `narrow` the remaining columns in one round of tiles of 192-wide footprint (TN =
// 6), which cost about three quarters of a whole tile each.  Every workgroup runs its share of the first walk and then
// of the second: no launch boundary and no waiting between them.  (`narrow` is never flipped: its columns are the
// caller's.)
template <typename T, bool A_KC, bool B_KC, int EPI>
__global__ __launch_bounds__(NT) void gemm_m16d_split_kernel(GemmProblem wide, GemmProblem narrow) {
  constexpr bool FLIP = A_KC && !B_KC;
  gemm_m16d_body<T, FLIP ? false : A_KC, FLIP ? true : B_KC, EPI, false, FLIP>(wide, TailShare{});
  // the second walk starts from scratch in LDS: every wave is done with the first walk's staging area
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  gemm_m16d_body<T, A_KC, B_KC, EPI, false, false, 6>(narrow, TailShare{});
}

#undef SRT_FENCE

// Host-side admission beyond the 32-deep kernel's: whole super-stages, at least four of them.
inline bool deep_fits(const GemmProblem& p) { return p.K % DK == 0 && p.K >= 4 * DK; }

template <typename T, bool A_KC, bool B_KC, int EPI, bool FLIP = false>
hipError_t launch_kernel(const GemmProblem& p, hipStream_t stream) {
  auto kernel = gemm_m16d_kernel<T, A_KC, B_KC, EPI, FLIP>;
  constexpr int lds_bytes = UNITS * UNIT;
  static std::atomic<uint32_t> configured{0};
  if (hipError_t e = ensure_lds_limit(reinterpret_cast<const void*>(kernel), lds_bytes, configured); e != hipSuccess) return e;
  const long long tiles = (long long)((p.M + 255) / 256) * ((p.N + BN - 1) / BN) * p.batch;
  const int grid = ring::persistent_grid(tiles);
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(NT), lds_bytes, stream, p);
  return launch_status(stream);
}

// The transposed product of `p` with the operands' roles exchanged and the result fields kept (see gemm_m16d_body, FLIP).
inline GemmProblem flipped(const GemmProblem& p) {
  GemmProblem q = p;
  q.M = p.N; q.N = p.M;
  q.A = p.B; q.sam = p.sbn; q.sak = p.sbk; q.sab = p.sbb;
  q.B = p.A; q.sbk = p.sak; q.sbn = p.sam; q.sbb = p.sab;
  return q;
}

// ---- the tail-sharing form ----------------------------------------------------------------------------
constexpr size_t TAIL_PARTIAL_BYTES = 256 * 256 * sizeof(float);   // per piece
constexpr size_t TAIL_FLAG_BYTES = 8192;                           // 255 x 3 flags (6120 bytes), ahead of the partials
constexpr size_t TAIL_STORED_OFFSET = 6144;                        // checking builds: 256 store counts behind the flags

// How the tail-sharing form would cut the left-over tiles of `p`; parts = 0: it does not apply.
struct TailPlan {
  int parts, cut1, cut2, groups, per_group;
  int left;          // tiles shared
  int tail_quads;    // length of the longest workgroup's share of them, in quads (a whole tile: K / 256)
};
inline TailPlan tail_plan(const GemmProblem& p) {
  TailPlan t{};
  if (!deep_fits(p) || p.K % (4 * DK) != 0) return t;
  const int grid = compute_units();
  if (grid % 8 != 0 || grid > 256) return t;
  const long long tiles = (long long)((p.M + 255) / 256) * ((p.N + BN - 1) / BN) * p.batch;
  const int left = (int)(tiles % grid), left8 = (left + 7) & ~7;
  const int Q = p.K / (4 * DK);
  if (left == 0 || tiles >= (1ll << 30)) return t;
  // Part 0 is made long enough to end after the others have published theirs (publishing costs about
  // what two quads of multiplying do), so that it finds their flags raised, publishes nothing and is the
  // only one to add up: pieces that end together would both publish and both add up.
  constexpr int PUB = 2;
  const int even = std::min(TAIL_MAX_PARTS, grid / left8);   // parts of one workgroup each
  if (even == 3 && Q >= 7) {
    t.parts = 3;
    t.cut1 = (Q + 2 * PUB + 2) / 3;
    t.cut2 = t.cut1 + (Q - t.cut1 + 1) / 2;
    t.groups = 2 * left8;
    t.per_group = 1;
  } else if (even >= 2 && Q >= 4) {
    t.parts = 2;
    t.cut1 = (Q + PUB + 1) / 2;
    t.cut2 = Q;
    t.groups = left8;
    t.per_group = 1;
  } else if (even < 2) {
    // two parts, the second short enough for a workgroup to take m of them in the time of a first part
    for (int m = 2; m <= 4 && t.parts == 0; ++m) {
      const int groups = ((left + m - 1) / m + 7) & ~7;
      const int cut = (m * (Q + PUB) + m) / (m + 1);   // ceil(m (Q + PUB) / (m + 1))
      if (left8 + groups <= grid && cut < Q) {
        t.parts = 2;
        t.cut1 = cut;
        t.cut2 = Q;
        t.groups = groups;
        t.per_group = m;
      }
    }
  }
  t.tail_quads = t.cut1 + 3;   // part 0 and its adding up (against quads per tile + 1 for a whole tile)
  t.left = left;
  return t;
}
inline bool tail_fits(const GemmProblem& p) { return tail_plan(p).parts != 0; }

template <typename T, bool A_KC, bool B_KC, int EPI, bool FLIP = false>
hipError_t launch_tail_kernel(const GemmProblem& p, hipStream_t stream) {
  auto kernel = gemm_m16d_tail_kernel<T, A_KC, B_KC, EPI, FLIP>;
  constexpr int lds_bytes = UNITS * UNIT;
  static std::atomic<uint32_t> configured{0};
  if (hipError_t e = ensure_lds_limit(reinterpret_cast<const void*>(kernel), lds_bytes, configured); e != hipSuccess) return e;
  const TailPlan plan = tail_plan(p);
  if (plan.parts == 0) return hipErrorInvalidValue;
  const int grid = compute_units();
  void* workspace = nullptr;
  // flags (and, in checking builds, the store counts behind them), then a partial per piece
  const size_t bytes = TAIL_FLAG_BYTES + (size_t)plan.left * plan.parts * TAIL_PARTIAL_BYTES;
  if (srtDeviceAllocate(&workspace, bytes, reinterpret_cast<srtStream>(stream)) != srtSuccess) return hipErrorOutOfMemory;
  TailShare ts;
  ts.parts = plan.parts;
  ts.cut1 = plan.cut1;
  ts.cut2 = plan.cut2;
  ts.groups = plan.groups;
  ts.per_group = plan.per_group;
  ts.flags = reinterpret_cast<unsigned long long*>(workspace);
  ts.stored = reinterpret_cast<unsigned int*>(static_cast<unsigned char*>(workspace) + TAIL_STORED_OFFSET);
  ts.partial = reinterpret_cast<float*>(static_cast<unsigned char*>(workspace) + TAIL_FLAG_BYTES);
  ts.epoch = next_launch_epoch();
#ifdef SRT_DEBUG_LAUNCH
  if (srtMemsetAsync(ts.stored, 0, 256 * sizeof(unsigned int), reinterpret_cast<srtStream>(stream)) != srtSuccess) {
    (void)srtDeviceFree(workspace);
    return hipErrorUnknown;
  }
#endif
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(NT), lds_bytes, stream, p, ts);
  hipError_t e = launch_status(stream);
#ifdef SRT_DEBUG_LAUNCH
  // (launch_status has waited for the kernel.)  No piece ever waits for another; what guarantees that some piece
  // of every shared tile adds up and stores is the order "publish, raise the flag, look at the others' flags" in
  // every piece.  Here that is checked: every left-over tile must have been stored at least once.
  if (e == hipSuccess) {
    unsigned int counts[256];
    e = hipMemcpyAsync(counts, ts.stored, sizeof(counts), hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    for (int i = 0; e == hipSuccess && i < plan.left; ++i)
      if (counts[i] == 0) e = hipErrorLaunchFailure;
  }
#endif
  (void)srtDeviceFree(workspace);   // stream-ordered: reused only by work queued after the kernel
  return e;
}

// (the transcendental activations have no tail-sharing form)
template <typename T, bool A_KC, bool B_KC>
hipError_t launch_tail(const GemmProblem& p, hipStream_t stream) {
  const bool trans = p.activation == srtActivationSigmoid || p.activation == srtActivationTanh ||
                     p.activation == srtActivationElu;
  if (trans) return hipErrorInvalidValue;
  // x . W as the transposed product, as in launch() -- from 96 tiles up: on a device a quarter full the flipped walk costs
  // more than the cheaper fragment reads give (1024 x 4096 x 4096, 64 tiles: 44.7 us against 44.1; 1536 x 4096 x 11008, 96
  // tiles: 112 against 115)
  if constexpr (A_KC && !B_KC) {
    const long long tiles = (long long)((p.M + 255) / 256) * ((p.N + BN - 1) / BN) * p.batch;
    if (tiles >= 96) {
      const GemmProblem q = flipped(p);
      if (p.activation == srtActivationClippedRelu) return launch_tail_kernel<T, false, true, EPI_CLIPPED, true>(q, stream);
      if (p.activation == srtActivationRelu) {
        if (p.bias) return launch_tail_kernel<T, false, true, EPI_BIAS_RELU, true>(q, stream);
        return launch_tail_kernel<T, false, true, EPI_RELU, true>(q, stream);
      }
      if (p.bias) return launch_tail_kernel<T, false, true, EPI_BIAS, true>(q, stream);
      return launch_tail_kernel<T, false, true, EPI_PLAIN, true>(q, stream);
    }
  }
  if (p.activation == srtActivationClippedRelu) return launch_tail_kernel<T, A_KC, B_KC, EPI_CLIPPED>(p, stream);
  if (p.activation == srtActivationRelu) {
    if (p.bias) return launch_tail_kernel<T, A_KC, B_KC, EPI_BIAS_RELU>(p, stream);
    return launch_tail_kernel<T, A_KC, B_KC, EPI_RELU>(p, stream);
  }
  if (p.bias) return launch_tail_kernel<T, A_KC, B_KC, EPI_BIAS>(p, stream);
  return launch_tail_kernel<T, A_KC, B_KC, EPI_PLAIN>(p, stream);
}

template <typename T, bool A_KC, bool B_KC>
hipError_t launch(const GemmProblem& p, hipStream_t stream) {
  // x . W runs as (W^T . x^T)^T: the flipped problem has an m-contiguous A and a k-contiguous B.  Whatever qualifies
  // this way round qualifies flipped: the operands' reaches and alignments exchange places, an n-contiguous B's N is a
  // multiple of 8 as an m-contiguous A's M must be, and the result is addressed as before.
  constexpr bool FLIP = A_KC && !B_KC;
  constexpr bool KA = FLIP ? false : A_KC, KB = FLIP ? true : B_KC;
  const GemmProblem q = FLIP ? flipped(p) : p;
  if (p.activation == srtActivationSigmoid) return launch_kernel<T, KA, KB, EPI_SIGMOID, FLIP>(q, stream);
  if (p.activation == srtActivationTanh) return launch_kernel<T, KA, KB, EPI_TANH, FLIP>(q, stream);
  if (p.activation == srtActivationElu) return launch_kernel<T, KA, KB, EPI_ELU, FLIP>(q, stream);
  if (p.activation == srtActivationClippedRelu) return launch_kernel<T, KA, KB, EPI_CLIPPED, FLIP>(q, stream);
  if (p.activation == srtActivationRelu) {
    if (p.bias) return launch_kernel<T, KA, KB, EPI_BIAS_RELU, FLIP>(q, stream);
    return launch_kernel<T, KA, KB, EPI_RELU, FLIP>(q, stream);
  }
  if (p.bias) return launch_kernel<T, KA, KB, EPI_BIAS, FLIP>(q, stream);
  return launch_kernel<T, KA, KB, EPI_PLAIN, FLIP>(q, stream);
}

// ---- the half tile ------------------------------------------------------------------------------------------------
template <typename T, bool B_KC, int EPI>
hipError_t launch_half_kernel(const GemmProblem& p, hipStream_t stream) {
  auto kernel = gemm_m16d_half_kernel<T, B_KC, EPI>;
  constexpr int lds_bytes = UNITS * UNIT;
  static std::atomic<uint32_t> configured{0};
  if (hipError_t e = ensure_lds_limit(reinterpret_cast<const void*>(kernel), lds_bytes, configured); e != hipSuccess) return e;
  const long long tiles = (long long)((p.M + 127) / 128) * ((p.N + BN - 1) / BN) * p.batch;
  const int grid = ring::persistent_grid(tiles);
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(NT), lds_bytes, stream, p);
  return launch_status(stream);
}

template <typename T, bool B_KC>
hipError_t launch_half(const GemmProblem& p, hipStream_t stream) {
  if (p.activation == srtActivationSigmoid) return launch_half_kernel<T, B_KC, EPI_SIGMOID>(p, stream);
  if (p.activation == srtActivationTanh) return launch_half_kernel<T, B_KC, EPI_TANH>(p, stream);
  if (p.activation == srtActivationElu) return launch_half_kernel<T, B_KC, EPI_ELU>(p, stream);
  if (p.activation == srtActivationClippedRelu) return launch_half_kernel<T, B_KC, EPI_CLIPPED>(p, stream);
  if (p.activation == srtActivationRelu) {
    if (p.bias) return launch_half_kernel<T, B_KC, EPI_BIAS_RELU>(p, stream);
    return launch_half_kernel<T, B_KC, EPI_RELU>(p, stream);
  }
  if (p.bias) return launch_half_kernel<T, B_KC, EPI_BIAS>(p, stream);
  return launch_half_kernel<T, B_KC, EPI_PLAIN>(p, stream);
}

// the 256 x 128 half tile (A not k-contiguous)
template <typename T, bool B_KC, int EPI>
hipError_t launch_narrow_kernel(const GemmProblem& p, hipStream_t stream) {
  auto kernel = gemm_m16d_narrow_kernel<T, B_KC, EPI>;
  constexpr int lds_bytes = UNITS * UNIT;
  static std::atomic<uint32_t> configured{0};
  if (hipError_t e = ensure_lds_limit(reinterpret_cast<const void*>(kernel), lds_bytes, configured); e != hipSuccess) return e;
  GemmProblem q = p;
  q.tile_n = 128;
  const long long tiles = (long long)((p.M + 255) / 256) * ((p.N + 127) / 128) * p.batch;
  const int grid = ring::persistent_grid(tiles);
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(NT), lds_bytes, stream, q);
  return launch_status(stream);
}

template <typename T, bool B_KC>
hipError_t launch_narrow(const GemmProblem& p, hipStream_t stream) {
  if (p.activation == srtActivationSigmoid) return launch_narrow_kernel<T, B_KC, EPI_SIGMOID>(p, stream);
  if (p.activation == srtActivationTanh) return launch_narrow_kernel<T, B_KC, EPI_TANH>(p, stream);
  if (p.activation == srtActivationElu) return launch_narrow_kernel<T, B_KC, EPI_ELU>(p, stream);
  if (p.activation == srtActivationClippedRelu) return launch_narrow_kernel<T, B_KC, EPI_CLIPPED>(p, stream);
  if (p.activation == srtActivationRelu) {
    if (p.bias) return launch_narrow_kernel<T, B_KC, EPI_BIAS_RELU>(p, stream);
    return launch_narrow_kernel<T, B_KC, EPI_RELU>(p, stream);
  }
  if (p.bias) return launch_narrow_kernel<T, B_KC, EPI_BIAS>(p, stream);
  return launch_narrow_kernel<T, B_KC, EPI_PLAIN>(p, stream);
}

// The split-K pass on half tiles (a k-contiguous A of at most 128 rows): fp32 accumulators to a workspace.
template <typename T, bool B_KC>
hipError_t launch_half_partial(const GemmProblem& p, hipStream_t stream) {
  return launch_half_kernel<T, B_KC, EPI_PARTIAL>(p, stream);
}

// ---- the split form: whole rounds of whole tiles, then one round of narrow tiles (gemm_m16d_split_kernel) ----------
// wide_cols = 0: the form does not apply.
struct SplitPlan {
  int wide_cols;   // columns of the first walk: whole 256-wide tiles that fill whole rounds of the grid
  int narrow_w;    // valid width of the second walk's tiles (a multiple of 8 in (128, 192])
  int grid;
};
inline SplitPlan split_plan(const GemmProblem& p) {
  SplitPlan s{0, 0, 0};
  const bool trans = p.activation == srtActivationSigmoid || p.activation == srtActivationTanh || p.activation == srtActivationElu;
  if (!deep_fits(p) || p.batch != 1 || trans) return s;
  const int grid = compute_units() & ~7;
  if (grid <= 0) return s;
  const long long tiles_m = (p.M + 255) / 256, cols = (p.N + 255) / 256;
  const long long rounds = tiles_m * cols / grid;        // whole rounds of whole tiles
  if (rounds < 1 || tiles_m * cols == rounds * grid || tiles_m > grid) return s;
  const long long c1 = rounds * grid / tiles_m;          // column tiles of the first walk (at most `rounds` rounds)
  const long long c2 = grid / tiles_m;                   // narrow tiles per row of tiles: one round holds them all
  const long long rest = p.N - 256 * c1;                 // columns left for the second walk
  if (c1 < 1 || rest <= 0) return s;
  const long long w = ((rest + c2 - 1) / c2 + 7) & ~7LL;
  // wider than 192: whole tiles lose nothing to speak of; up to 128: a tile half as wide would be the one (not built)
  if (w > 192 || w <= 128) return s;
  s.wide_cols = (int)(256 * c1);
  s.narrow_w = (int)w;
  s.grid = grid;
  return s;
}
inline bool split_fits(const GemmProblem& p) { return split_plan(p).wide_cols != 0; }

template <typename T, bool A_KC, bool B_KC, int EPI>
hipError_t launch_split_kernel(const GemmProblem& p, hipStream_t stream) {
  auto kernel = gemm_m16d_split_kernel<T, A_KC, B_KC, EPI>;
  constexpr int lds_bytes = UNITS * UNIT;
  static std::atomic<uint32_t> configured{0};
  if (hipError_t e = ensure_lds_limit(reinterpret_cast<const void*>(kernel), lds_bytes, configured); e != hipSuccess) return e;
  const SplitPlan plan = split_plan(p);
  if (plan.wide_cols == 0) return hipErrorInvalidValue;
  auto at = [](const void* base, long long elements) {
    return static_cast<const void*>(static_cast<const char*>(base) + elements * 2);   // 16-bit elements
  };
  GemmProblem wide = p, narrow = p;
  wide.N = plan.wide_cols;
  narrow.N = p.N - plan.wide_cols;
  narrow.tile_n = plan.narrow_w;
  narrow.B = at(p.B, (long long)plan.wide_cols * p.sbn);
  narrow.C = const_cast<void*>(at(p.C, (long long)plan.wide_cols * p.scn));
  if (p.bias && !p.bias_per_row) narrow.bias = at(p.bias, (long long)plan.wide_cols * p.sbias);
  constexpr bool FLIP = A_KC && !B_KC;
  const GemmProblem first = FLIP ? flipped(wide) : wide;
  hipLaunchKernelGGL(kernel, dim3(plan.grid), dim3(NT), lds_bytes, stream, first, narrow);
  return launch_status(stream);
}

// (the transcendental activations have no split form)
template <typename T, bool A_KC, bool B_KC>
hipError_t launch_split(const GemmProblem& p, hipStream_t stream) {
  if (p.activation == srtActivationClippedRelu) return launch_split_kernel<T, A_KC, B_KC, EPI_CLIPPED>(p, stream);
  if (p.activation == srtActivationRelu) {
    if (p.bias) return launch_split_kernel<T, A_KC, B_KC, EPI_BIAS_RELU>(p, stream);
    return launch_split_kernel<T, A_KC, B_KC, EPI_RELU>(p, stream);
  }
  if (p.bias) return launch_split_kernel<T, A_KC, B_KC, EPI_BIAS>(p, stream);
  return launch_split_kernel<T, A_KC, B_KC, EPI_PLAIN>(p, stream);
}

// The split-K pass: fp32 accumulators to a workspace, no epilogue arithmetic.
template <typename T, bool A_KC, bool B_KC>
hipError_t launch_partial(const GemmProblem& p, hipStream_t stream) {
  return launch_kernel<T, A_KC, B_KC, EPI_PARTIAL>(p, stream);
}

}  // namespace m16d
}  // namespace srt
