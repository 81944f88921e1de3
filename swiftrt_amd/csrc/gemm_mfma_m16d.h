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
template <bool KC>
struct Loader {
  uint32_t voff[KC ? 2 : 4];
  static constexpr int SOFFS = KC ? 4 : 2;
  static constexpr int vindex(int i) { return KC ? (i & 1) : (i & 3); }
  static constexpr int sindex(int i) { return KC ? (i >> 1) : (i >> 2); }
  static constexpr uint32_t landing(int i) { return KC ? (uint32_t)i * 1024u : (uint32_t)(i >> 2) * 16384u + (uint32_t)(i & 3) * 1024u; }
  static __device__ __forceinline__ uint32_t wave_share(int wave) { return (uint32_t)wave * (KC ? 8192u : 4096u); }
  // bytes between so[j] and so[j + 1]: 16 rows (KC) or 32 k rows (MN)
  static __device__ __forceinline__ uint32_t step(long long ld) { return (uint32_t)((KC ? 16 : 32) * ld * 2); }

  // ld: elements between rows (KC) or between k (MN)
  __device__ __forceinline__ void init(int wave, int lane, long long ld) {
    if constexpr (KC) {
      // load i covers rows (8 wave + i) 8 .. + 7, 8 lanes per 128-byte row; (row >> 1) & 7 depends on the
      // lane and the parity of i only, so loads i and i + 2 differ by 16 rows in the scalar offset
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int row = (wave * 8 + i) * 8 + (lane >> 3);
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

template <typename T, bool A_KC, bool B_KC, int EPI>
__global__ __launch_bounds__(NT) void gemm_m16d_kernel(GemmProblem p) {
  constexpr int TM = 8;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[];
  const uint32_t lds = (uint32_t)(uintptr_t)(SRT_LDS unsigned char*)lds_raw;
  const uint32_t lds_end = lds + UNITS * UNIT;

  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  auto lane_id = []() {
    uint32_t zero = 0;
    asm volatile("" : "+s"(zero));   // opaque: keeps the two instructions where they are written
    return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, zero));
  };
  const int wm0 = (wave >> 1) * 128, wn0 = (wave & 1) * 128;

  const int tiles_m = (p.M + 255) / 256, tiles_n = (p.N + BN - 1) / BN;
  const int total = tiles_m * tiles_n * p.batch;
  const int grid = (int)gridDim.x;
  int v = (int)blockIdx.x;

  const long long lda = A_KC ? p.sam : p.sak;
  const long long ldb = B_KC ? p.sbn : p.sbk;
  const long long a_view = A_KC ? (long long)(p.M - 1) * lda + p.K : (long long)(p.K - 1) * lda + p.M;
  const long long b_view = B_KC ? (long long)(p.N - 1) * ldb + p.K : (long long)(p.K - 1) * ldb + p.N;
  const u32x4_t ra = ring::make_rsrc(p.A, (uint32_t)(((long long)(p.batch - 1) * p.sab + a_view) * 2));
  const u32x4_t rb = ring::make_rsrc(p.B, (uint32_t)(((long long)(p.batch - 1) * p.sbb + b_view) * 2));
  const uint32_t kstep_a = A_KC ? (uint32_t)(DK * 2) : (uint32_t)(DK * lda * 2);   // bytes per super-stage
  const uint32_t kstep_b = B_KC ? (uint32_t)(DK * 2) : (uint32_t)(DK * ldb * 2);
  const uint32_t lstep_a = Loader<A_KC>::step(lda), lstep_b = Loader<B_KC>::step(ldb);
  const int S = p.K / DK;   // super-stages per tile (the host admits whole ones only, at least four)

  // per-XCD start of the k walk for an A stored k x m (see gemm_ring_kernel)
#ifndef SRT_M16D_ROTATE   // measurement builds: 0 never, 1 always
  constexpr bool rotate = !A_KC;
#else
  constexpr bool rotate = SRT_M16D_ROTATE != 0;
#endif
  const int rot = rotate ? (int)(((unsigned)(blockIdx.x & 7) * (unsigned)S) / 8u) : 0;
  auto stage_of = [&](int r) {
    int e = r + rot;
    e = e >= S ? e - S : e;
    e = e >= S ? e - S : e;
    return e;
  };
  auto wrap = [&](uint32_t a) { return a >= lds_end ? a - UNITS * UNIT : a; };

  TileRef cur_tile = m16::locate_tile<A_KC, B_KC, 256>(p, v, tiles_m, tiles_n);

  // the eight loads of one unit, outside the main loop (first fill, and B_1 after an epilogue)
  auto issue_a = [&](const Loader<A_KC>& l, uint32_t slot, uint32_t base) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      ring::load_to_lds(ra, slot + Loader<A_KC>::wave_share(wave) + Loader<A_KC>::landing(i),
                        l.voff[Loader<A_KC>::vindex(i)], base + (uint32_t)Loader<A_KC>::sindex(i) * lstep_a);
  };
  auto issue_b = [&](const Loader<B_KC>& l, uint32_t slot, uint32_t base) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      ring::load_to_lds(rb, slot + Loader<B_KC>::wave_share(wave) + Loader<B_KC>::landing(i),
                        l.voff[Loader<B_KC>::vindex(i)], base + (uint32_t)Loader<B_KC>::sindex(i) * lstep_b);
  };

  uint32_t x = lds;   // slot of A_s; B_s follows it, then A_{s+1}, B_{s+1}, A_{s+2} (B_{s+2} goes where A_s is)

  bool first_tile = true;
  for (;;) {
    // per-lane addressing state, derived per tile and scoped to it (see gemm_ring_kernel)
    Loader<A_KC> la;
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
      asm volatile("s_waitcnt vmcnt(16)\n\ts_barrier" ::: "memory");
    } else {
      issue_b(lb, xb1, cur_tile.offb + (uint32_t)stage_of(1) * kstep_b);
    }
    first_tile = false;
    SRT_FENCE();

    const int vn = v + grid;
    const bool has_next = vn < total;
    const TileRef next_tile =
        m16::locate_tile<A_KC, B_KC, 256>(p, (int)select_lt(vn, total, (uint32_t)vn, (uint32_t)v), tiles_m, tiles_n);
    // A requests below limit_a are real (A'_0 and A'_1 of the next tile); of B only B'_0: B'_1 would land in
    // the staging area
    const int limit_a = (int)select_lt(vn, total, (uint32_t)(S + 2), (uint32_t)S);
    const int limit_b = (int)select_lt(vn, total, (uint32_t)(S + 1), (uint32_t)S);

    f32x4_t acc[TM][8];   // defined by the MFMAs of the tile's first super-stage
    u32x4_t af[TM], bf[8];
#pragma unroll
    for (int t = 0; t < 4; ++t) bf[t] = fb.template read<0>(xb, t);
#pragma unroll
    for (int t = 0; t < 4; ++t) af[t] = fa.template read<0>(x, t);

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
#pragma unroll
      for (int j = 0; j < 8; ++j) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int u = 4 * j + i;
          // which load, if any, rides on this MFMA
          const int ld = LOADS == 3 ? ((u & 3) == 0 ? u >> 2 : -1)
                       : (LOADS == 1 || LOADS == 2) ? ((u >= 16 && (u & 3) == 0) ? ((u - 16) >> 2) + (LOADS == 2 ? 4 : 0) : -1)
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
              constexpr uint32_t imm[8] = {Loader<A_KC>::landing(0), Loader<A_KC>::landing(1), Loader<A_KC>::landing(2),
                                           Loader<A_KC>::landing(3), Loader<A_KC>::landing(4), Loader<A_KC>::landing(5),
                                           Loader<A_KC>::landing(6), Loader<A_KC>::landing(7)};
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
#ifdef SRT_M16D_SWAP_OPERANDS   // measurement builds: A fragment first (accumulator tiles come out untransposed)
          if constexpr (FIRST) mfma16_first<T>(acc[4 * AH + i][j], af[4 * AH + i], bf[j]);
          else mfma16<T>(acc[4 * AH + i][j], af[4 * AH + i], bf[j]);
#else
          if constexpr (FIRST) mfma16_first<T>(acc[4 * AH + i][j], bf[j], af[4 * AH + i]);
          else mfma16<T>(acc[4 * AH + i][j], bf[j], af[4 * AH + i]);
#endif
          if (ld >= 0) {
            SRT_FENCE();
            const int si = LOADS == 3 ? Loader<B_KC>::sindex(ld) : Loader<A_KC>::sindex(ld);
            const uint32_t so = si == 0 ? so0 : si == 1 ? so1 : si == 2 ? so2 : so3;
            if (LOADS == 3) ring::load_to_lds_at_m0(rb, lb.voff[Loader<B_KC>::vindex(ld)], so);
            else ring::load_to_lds_at_m0(ra, la.voff[Loader<A_KC>::vindex(ld)], so);
          }
          if (!(SRT_ABLATE & 4) || FIRST) {   // (measurement builds can keep the first super-stage's fragments)
            if (OWN) {
              if (u < 8 && (u & 1) == 0) bf[4 + (u >> 1)] = fb.template read<H>(ub, 4 + (u >> 1));
              if (u >= 8 && u < 16 && (u & 1) == 0) af[4 + ((u - 8) >> 1)] = fa.template read<H>(ua, 4 + ((u - 8) >> 1));
            } else {
              if (u < 16 && (u & 3) == 1) af[u >> 2] = fa.template read<H>(ua, u >> 2);
              if (u < 16 && (u & 3) == 3) bf[u >> 2] = fb.template read<H>(ub, u >> 2);
            }
          }
          ev(u);
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
        if (u == 9) ta = xa2 + Loader<A_KC>::wave_share(wave);
        if (u == 11) so_a0 = soa;
        if (u == 13) so_a1 = select_lt(r, limit_a, soa + lstep_a, OOB);
      });
      // ---- phase 1: k half 0, A tiles 4-7; loads 4-7 of A_{s+2}; reads of k half 1 ----
      phase(C1{}, first_tag, std::false_type{}, C1{}, C2{}, x, xb, ta, so_a0, so_a1, so_a2, so_a3, [&](int u) __attribute__((always_inline)) {
        if (Loader<A_KC>::SOFFS == 4) {
          if (u == 2) so_a2 = select_lt(r, limit_a, soa + 2 * lstep_a, OOB);
          if (u == 6) so_a3 = select_lt(r, limit_a, soa + 3 * lstep_a, OOB);
        }
        if (u == 10) sel = select_lt(r, S, cur_tile.offb, next_tile.offb);
        if (u == 14) sob = select_lt(r, limit_b, sel + eb_off, OOB);
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
      if (SRT_ABLATE & 1) asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");
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
    const int em0 = cur_tile.m0 + wm0, en0 = cur_tile.n0 + wn0, bz = cur_tile.bz;
    const int le = lane_id();
    constexpr bool LINEAR_BIAS = EPI == EPI_BIAS || EPI == EPI_BIAS_RELU || EPI == EPI_CLIPPED;
    u32x2_t bias_regs[8];
    if (LINEAR_BIAS) m16::load_bias<T, TM>(p, em0, en0, le, bias_regs);   // lands during the wait below
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier\n\ts_nop 7\n\ts_nop 7" ::: "memory");
    if (LINEAR_BIAS) m16::pin_all<TM>(acc);
    // staging: the slots of A_{S-1} (waves 0, 1) and B_{S-1} (waves 2, 3), half a slot each; x is A_S's by now
    uint32_t sa = x < lds + 2 * UNIT ? x + 3 * UNIT : x - 2 * UNIT;
    uint32_t sb = x < lds + UNIT ? x + 4 * UNIT : x - UNIT;
    const uint32_t stage = ((wave & 2) ? sb : sa) + (uint32_t)(wave & 1) * (uint32_t)(UNIT / 2);

    if (EPI == EPI_PARTIAL) {
      m16::store_tile_partial<TM>(p, acc, em0, en0, bz, le, stage);
    } else if (EPI == EPI_TRANS) {
      m16::load_bias<T, TM>(p, em0, en0, le, bias_regs);
      m16::store_tile_transcendental<T, TM>(p, acc, em0, en0, bz, le, stage, bias_regs);
    } else {
      if (EPI == EPI_BIAS) m16::store_tile<T, TM, true, 0>(p, acc, em0, en0, bz, le, stage, bias_regs);
      else if (EPI == EPI_RELU) m16::store_tile<T, TM, false, 1>(p, acc, em0, en0, bz, le, stage, bias_regs);
      else if (EPI == EPI_BIAS_RELU) m16::store_tile<T, TM, true, 1>(p, acc, em0, en0, bz, le, stage, bias_regs);
      else if (EPI == EPI_CLIPPED) m16::store_tile<T, TM, true, 2>(p, acc, em0, en0, bz, le, stage, bias_regs);
      else m16::store_tile<T, TM, false, 0>(p, acc, em0, en0, bz, le, stage, bias_regs);
    }
    if (!has_next) break;

    // every wave has finished reading its staging area before any wave's loads overwrite it
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    v = vn;
    cur_tile = next_tile;
  }
}

#undef SRT_FENCE

// Host-side admission beyond the 32-deep kernel's: whole super-stages, at least four of them.
inline bool deep_fits(const GemmProblem& p) { return p.K % DK == 0 && p.K >= 4 * DK; }

template <typename T, bool A_KC, bool B_KC, int EPI>
hipError_t launch_kernel(const GemmProblem& p, hipStream_t stream) {
  auto kernel = gemm_m16d_kernel<T, A_KC, B_KC, EPI>;
  constexpr int lds_bytes = UNITS * UNIT;
  static std::atomic<uint32_t> configured{0};
  if (hipError_t e = ensure_lds_limit(reinterpret_cast<const void*>(kernel), lds_bytes, configured); e != hipSuccess) return e;
  const long long tiles = (long long)((p.M + 255) / 256) * ((p.N + BN - 1) / BN) * p.batch;
  const int grid = ring::persistent_grid(tiles);
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(NT), lds_bytes, stream, p);
  return launch_status(stream);
}

template <typename T, bool A_KC, bool B_KC>
hipError_t launch(const GemmProblem& p, hipStream_t stream) {
  const bool trans = p.activation == srtActivationSigmoid || p.activation == srtActivationTanh ||
                     p.activation == srtActivationElu;
  if (trans) return launch_kernel<T, A_KC, B_KC, EPI_TRANS>(p, stream);
  if (p.activation == srtActivationClippedRelu) return launch_kernel<T, A_KC, B_KC, EPI_CLIPPED>(p, stream);
  if (p.activation == srtActivationRelu) {
    if (p.bias) return launch_kernel<T, A_KC, B_KC, EPI_BIAS_RELU>(p, stream);
    return launch_kernel<T, A_KC, B_KC, EPI_RELU>(p, stream);
  }
  if (p.bias) return launch_kernel<T, A_KC, B_KC, EPI_BIAS>(p, stream);
  return launch_kernel<T, A_KC, B_KC, EPI_PLAIN>(p, stream);
}

}  // namespace m16d
}  // namespace srt
