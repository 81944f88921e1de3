// 128 x 128 bf16 / fp16 matmul tile kernel for gfx950 on v_mfma_f32_16x16x32: the quarter tile of the 64-deep
// 256 x 256 kernel (gemm_mfma_m16d.h), for problems whose whole or half tiles would leave most compute units
// without work -- 1024 x 4096 (x 4096 deep) is 64 whole tiles or 128 half tiles on 256 units, and 256 of these.
//
// What is kept: direct-to-LDS loads of whole cache lines, a ring of five 32 KiB slots (the whole LDS), requests two
// super-stages ahead, one barrier per super-stage, the persistent XCD-aware tile walk that runs on across tile
// boundaries, MFMAs written out with the accumulators tied, the epilogue (m16::store_tile on a 4 x 4 block).
// What differs: the wave tile is 64 x 64 (4 x 4 MFMA tiles, 64 accumulator registers), so a 32-deep slice of k is only
// 16 MFMAs = 256 cycles, and two things follow.
//   * A unit of staging is 128 rows (or columns) x 128 k = 32 KiB, twice as deep as the 256-wide kernels': a
//     super-stage -- four slices, 64 MFMAs per wave -- then lasts as long as the 128 x 256 half tile's, and two of them
//     cover the load latency.  K must be a multiple of 128 and at least 256 (with two or three units per tile every
//     request of the main loop already belongs to the workgroup's next tile).
//   * The fragments of a slice cannot wait for registers to fall free inside it (the 256-wide kernels re-read each
//     B tile "right behind its last MFMA", 32 MFMAs ahead of its next use; here that would be 8).  There are
//     registers to spare instead: two fragment sets, the next slice's eight fragments read into the idle set while
//     this slice multiplies.
// Layouts of a unit (both [128][16 chunks of 16 B], 256 B = every LDS bank once per row):
//   k-contiguous operand:  row r = m (n), chunk c = k / 8, at position c ^ (r & 15): a 16 x 32 fragment is one
//                          ds_read_b128 whose sixteen lanes of a group hit sixteen different chunks.
//   mn-contiguous operand: row = k, chunk c = m / 8, at position c ^ ((k & 3) << 2) ^ (((k >> 3) & 1) << 1): the
//                          32-deep kernel's swizzle on rows half as long; fragments by ds_read_b64_tr_b16 pairs.
// A load instruction moves 4 rows x 256 B; a wave issues eight per unit (rows 32 wave + 4 i ..): the per-lane offset
// depends on i mod 4 only and loads i and i + 4 differ by 16 rows in the scalar offset.
// Schedule of super-stage s (slices 0-3 of units A_s, B_s; fragment set = slice mod 2):
//   slice 0      scalar bookkeeping for the request of A_{s+2}; reads slice 1
//   slice 1, 2   the eight loads of A_{s+2} (into the slot of B_{s-1}); read slices 2, 3
//   sync         s_waitcnt vmcnt(8) lgkmcnt(0); s_barrier: all of super-stage s is in registers, A_{s+1} and
//                B_{s+1} have landed for every wave
//   slice 3      the eight loads of B_{s+2} (into the slot of A_s); reads slice 0 of super-stage s + 1
#pragma once
#include "gemm_mfma_m16d.h"

namespace srt {
namespace m16q {

using m16::EPI_BIAS;
using m16::EPI_BIAS_RELU;
using m16::EPI_CLIPPED;
using m16::EPI_ELU;
using m16::EPI_PLAIN;
using m16::EPI_RELU;
using m16::EPI_SIGMOID;
using m16::EPI_TANH;
using m16::mfma16;
using m16::mfma16_first;
using m16d::select_lt;
using ring::BN;
using ring::f32x4_t;
using ring::NT;
using ring::OOB;
using ring::s16x4_t;
using ring::TileRef;
using ring::u32x2_t;
using ring::u32x4_t;

#define SRT_FENCE() __builtin_amdgcn_sched_barrier(0)

constexpr int TILE = 128;            // rows and columns of a workgroup tile
constexpr int DK = 128;              // k depth of a unit
constexpr int UNIT = TILE * DK * 2;  // bytes of a unit: 32 KiB
constexpr int UNITS = 5;             // slots: the whole LDS

// ---- global -> LDS: eight loads per wave and unit ----------------------------------------------------
// Load i takes lane offset voff[i & 3], scalar offset so[i >> 2] (so[1] = so[0] + step) and lands i KiB into the
// wave's 8 KiB of the slot.
template <bool KC>
struct Loader {
  uint32_t voff[4];
  static constexpr int vindex(int i) { return i & 3; }
  static constexpr int sindex(int i) { return i >> 2; }
  static constexpr uint32_t landing(int i) { return (uint32_t)i * 1024u; }
  static __device__ __forceinline__ uint32_t wave_share(int wave) { return (uint32_t)wave * 8192u; }
  // bytes between so[0] and so[1]: 16 rows
  static __device__ __forceinline__ uint32_t step(long long ld) { return (uint32_t)(16 * ld * 2); }

  // ld: elements between rows (KC: rows are m or n; MN: rows are k)
  __device__ __forceinline__ void init(int wave, int lane, long long ld) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = wave * 32 + i * 4 + (lane >> 4);   // + 16 for loads 4-7: the swizzles do not see bit 4
      const int swz = KC ? (row & 15) : (((row & 3) << 2) ^ (((row >> 3) & 1) << 1));
      const int chunk = (lane & 15) ^ swz;
      voff[i] = (uint32_t)(((long long)row * ld + chunk * 8) * 2);
    }
  }
};

// ---- LDS -> MFMA operands: 16 rows x 32 k of slice Q ---------------------------------------------------
template <bool KC>
struct FragReader;
template <>
struct FragReader<true> {
  uint32_t off[4];   // per slice; tile t adds t * 4096
  __device__ __forceinline__ void init(int lane, int wave_row0) {
    const int g = lane >> 4, jn = lane & 15;   // (row & 15 = jn: wave_row0 is a multiple of 16)
#pragma unroll
    for (int q = 0; q < 4; ++q) off[q] = (uint32_t)((wave_row0 + jn) * 256 + (((4 * q + g) ^ jn) << 4));
  }
  template <int Q>
  __device__ __forceinline__ u32x4_t read(uint32_t unit, int t) const {
    return *reinterpret_cast<const SRT_LDS u32x4_t*>(unit + off[Q] + t * 4096);
  }
};
template <>
struct FragReader<false> {
  uint32_t off[4];   // per tile; slice q adds q * 8192
  __device__ __forceinline__ void init(int lane, int wave_row0) {
    // lane supplies the address of T[k = 8 g + e (+ 4 for the second read)][mn = wave_row0 + 16 t + 4 q]
    const int g = lane >> 4, jn = lane & 15;
    const int e = jn >> 2, q = jn & 3;
    const int krow = 8 * g + e;
    const int mn = wave_row0 + 4 * q;   // tile t adds 16: two 16-byte chunks
    const uint32_t base = (uint32_t)(krow * 256 + ((mn >> 2) & 1) * 8);
    const int chunk0 = mn >> 3, swz = (e << 2) ^ ((g & 1) << 1);   // k & 3 = e, bit 3 of k = g & 1
#pragma unroll
    for (int t = 0; t < 4; ++t) off[t] = base + (uint32_t)(((chunk0 + 2 * t) ^ swz) << 4);
  }
  template <int Q>
  __device__ __forceinline__ u32x4_t read(uint32_t unit, int t) const {
    const uint32_t a = unit + off[t] + Q * 8192;
    const u32x2_t lo =
        __builtin_bit_cast(u32x2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<SRT_LDS s16x4_t*>(a)));
    const u32x2_t hi = __builtin_bit_cast(
        u32x2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<SRT_LDS s16x4_t*>(a + 1024)));
    u32x4_t v = {lo.x, lo.y, hi.x, hi.y};
    return v;
  }
};

template <typename T, bool A_KC, bool B_KC, int EPI>
__device__ __forceinline__ void gemm_m16q_body(const GemmProblem& p) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[];
  const uint32_t lds = (uint32_t)(uintptr_t)(SRT_LDS unsigned char*)lds_raw;
  const uint32_t lds_end = lds + UNITS * UNIT;

  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  auto lane_id = []() {
    uint32_t zero = 0;
    asm volatile("" : "+s"(zero));   // opaque: keeps the two instructions where they are written
    return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, zero));
  };
  const int wm0 = (wave >> 1) * 64, wn0 = (wave & 1) * 64;

  const int tiles_m = (p.M + TILE - 1) / TILE, tiles_n = (p.N + TILE - 1) / TILE;
  const int total = tiles_m * tiles_n * p.batch;
  const int grid = (int)gridDim.x;
  int v = (int)blockIdx.x;
  if (v >= total) return;

  const long long lda = A_KC ? p.sam : p.sak;
  const long long ldb = B_KC ? p.sbn : p.sbk;
  const long long a_view = A_KC ? (long long)(p.M - 1) * lda + p.K : (long long)(p.K - 1) * lda + p.M;
  const long long b_view = B_KC ? (long long)(p.N - 1) * ldb + p.K : (long long)(p.K - 1) * ldb + p.N;
  const u32x4_t ra = ring::make_rsrc(p.A, (uint32_t)(((long long)(p.batch - 1) * p.sab + a_view) * 2));
  const u32x4_t rb = ring::make_rsrc(p.B, (uint32_t)(((long long)(p.batch - 1) * p.sbb + b_view) * 2));
  // tile number -> position and operand offsets (the walk's own columns are 256 apart)
  auto locate = [&](int tile) {
    TileRef t = m16::locate_tile<A_KC, B_KC, TILE>(p, tile, tiles_m, tiles_n);
    t.n0 = (t.n0 / BN) * TILE;
    t.offb = (uint32_t)(((long long)t.bz * p.sbb + (B_KC ? (long long)t.n0 * ldb : (long long)t.n0)) * 2);
    return t;
  };
  const uint32_t kstep_a = A_KC ? (uint32_t)(DK * 2) : (uint32_t)(DK * lda * 2);   // bytes per super-stage
  const uint32_t kstep_b = B_KC ? (uint32_t)(DK * 2) : (uint32_t)(DK * ldb * 2);
  const uint32_t lstep_a = Loader<A_KC>::step(lda), lstep_b = Loader<B_KC>::step(ldb);
  const int S = p.K / DK;   // super-stages per tile (the host admits whole ones only, at least two)

  // per-XCD start of the k walk for an A stored k x m (see gemm_ring_kernel)
  const int rot = !A_KC ? (int)(((unsigned)(blockIdx.x & 7) * (unsigned)S) / 8u) : 0;
  auto stage_of = [&](int r) {   // r = 0, 1, 2 only
    int e = r + rot;
    e = e >= S ? e - S : e;
    e = e >= S ? e - S : e;
    return e;
  };
  auto wrap = [&](uint32_t a) { return a >= lds_end ? a - UNITS * UNIT : a; };

  TileRef cur_tile = locate(v);

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
    const TileRef next_tile = locate((int)select_lt(vn, total, (uint32_t)vn, (uint32_t)v));
    // A requests below limit_a are real (A'_0 and A'_1 of the next tile); of B only B'_0: B'_1 would land in
    // the staging area
    const int limit_a = (int)select_lt(vn, total, (uint32_t)(S + 2), (uint32_t)S);
    const int limit_b = (int)select_lt(vn, total, (uint32_t)(S + 1), (uint32_t)S);

    f32x4_t acc[4][4];   // defined by the MFMAs of the tile's first slice (every slice multiplies into all sixteen)
    u32x4_t af[2][4], bf[2][4];
#pragma unroll
    for (int t = 0; t < 4; ++t) bf[0][t] = fb.template read<0>(xb, t);
#pragma unroll
    for (int t = 0; t < 4; ++t) af[0][t] = fa.template read<0>(x, t);

    int e_req = stage_of(2);   // k index of request s + 2
    uint32_t ea_off = (uint32_t)e_req * kstep_a, eb_off = (uint32_t)e_req * kstep_b;

    auto set_target = [](auto imm_tag, uint32_t base) __attribute__((always_inline)) {
      ring::set_lds_target<decltype(imm_tag)::value>(base);
    };

    // One slice: 16 MFMAs, B tile by B tile (u = 4 j + i), on fragment set CUR; the eight fragments of slice NQ of
    // the units (ua, ub) are read into the other set, in the order of their first use (b0 a0 a1 a2 a3 b1 b2 b3),
    // one behind every other MFMA.
    //   LOADS 0: none; 1: A loads 0-3; 2: A loads 4-7; 3: B loads 0-7 -- `target`: the request's slot plus the wave's
    //   share, so0 / so1: its scalar offsets.  `ev(u)`: scalar bookkeeping.
    auto slice = [&](auto cur_tag, auto first_tag, auto nq_tag, auto loads_tag, uint32_t ua, uint32_t ub,
                     const uint32_t& target, const uint32_t& so0, const uint32_t& so1, auto&& ev) __attribute__((always_inline)) {
      constexpr int CUR = decltype(cur_tag)::value, NXT = CUR ^ 1;
      constexpr bool FIRST = decltype(first_tag)::value;
      constexpr int NQ = decltype(nq_tag)::value;
      constexpr int LOADS = decltype(loads_tag)::value;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int u = 4 * j + i;
          const int ld = LOADS == 3 ? ((u & 1) == 1 ? u >> 1 : -1)
                       : (LOADS == 1 || LOADS == 2) ? ((u & 3) == 1 ? (u >> 2) + (LOADS == 2 ? 4 : 0) : -1)
                       : -1;
          if (ld >= 0) {
            if (ld == 0) set_target(std::integral_constant<uint32_t, 0u>{}, target);
            if (ld == 1) set_target(std::integral_constant<uint32_t, 1024u>{}, target);
            if (ld == 2) set_target(std::integral_constant<uint32_t, 2048u>{}, target);
            if (ld == 3) set_target(std::integral_constant<uint32_t, 3072u>{}, target);
            if (ld == 4) set_target(std::integral_constant<uint32_t, 4096u>{}, target);
            if (ld == 5) set_target(std::integral_constant<uint32_t, 5120u>{}, target);
            if (ld == 6) set_target(std::integral_constant<uint32_t, 6144u>{}, target);
            if (ld == 7) set_target(std::integral_constant<uint32_t, 7168u>{}, target);
            SRT_FENCE();
          }
          if constexpr (FIRST) mfma16_first<T>(acc[i][j], bf[CUR][j], af[CUR][i]);
          else mfma16<T>(acc[i][j], bf[CUR][j], af[CUR][i]);
          if (ld >= 0) {
            SRT_FENCE();
            const uint32_t so = (ld >> 2) == 0 ? so0 : so1;
            if (LOADS == 3) ring::load_to_lds_at_m0(rb, lb.voff[ld & 3], so);
            else ring::load_to_lds_at_m0(ra, la.voff[ld & 3], so);
          }
          if ((u & 1) == 0) {
            const int f = u >> 1;
            if (f == 0) bf[NXT][0] = fb.template read<NQ>(ub, 0);
            else if (f <= 4) af[NXT][f - 1] = fa.template read<NQ>(ua, f - 1);
            else bf[NXT][f - 4] = fb.template read<NQ>(ub, f - 4);
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
      uint32_t so_a0 = OOB, so_a1 = OOB, so_b0 = OOB, so_b1 = OOB;
      // ---- slice 0: the request of A_{s+2} is worked out ----
      slice(C0{}, first_tag, C1{}, C0{}, x, xb, ta, so_a0, so_a1, [&](int u) __attribute__((always_inline)) {
        if (u == 1) xa2 = xa1 + 2 * UNIT;
        if (u == 3) xa2 = select_lt((int)xa2, (int)lds_end, xa2, xa2 - UNITS * UNIT);
        if (u == 5) sel = select_lt(r, S, cur_tile.offa, next_tile.offa);
        if (u == 7) soa = select_lt(r, limit_a, sel + ea_off, OOB);
        if (u == 9) ta = xa2 + Loader<A_KC>::wave_share(wave);
        if (u == 11) so_a0 = soa;
        if (u == 13) so_a1 = select_lt(r, limit_a, soa + lstep_a, OOB);
      });
      // ---- slice 1: loads 0-3 of A_{s+2} ----
      slice(C1{}, std::false_type{}, C2{}, C1{}, x, xb, ta, so_a0, so_a1, [&](int u) __attribute__((always_inline)) {
        if (u == 3) sel = select_lt(r, S, cur_tile.offb, next_tile.offb);
        if (u == 7) sob = select_lt(r, limit_b, sel + eb_off, OOB);
      });
      // ---- slice 2: loads 4-7 of A_{s+2} ----
      slice(C0{}, std::false_type{}, C3{}, C2{}, x, xb, ta, so_a0, so_a1, [&](int u) __attribute__((always_inline)) {
        if (u == 3) so_b0 = sob;
        if (u == 7) so_b1 = select_lt(r, limit_b, sob + lstep_b, OOB);
        if (u == 11) tb = x + Loader<B_KC>::wave_share(wave);
      });
      // ---- sync: all of super-stage s is in registers, A_{s+1} and B_{s+1} have landed ----
      asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      SRT_FENCE();
      // ---- slice 3: the loads of B_{s+2}; reads of super-stage s + 1 ----
      slice(C1{}, std::false_type{}, C0{}, C3{}, xa1, xb1, tb, so_b0, so_b1, [&](int u) __attribute__((always_inline)) {
        // the next request's k index: one further, or back to 0 past the tile's last super-stage
        if (u == 2) ea_off = select_lt(e_req + 1, S, ea_off + kstep_a, 0u);
        if (u == 6) eb_off = select_lt(e_req + 1, S, eb_off + kstep_b, 0u);
        if (u == 10) e_req = (int)select_lt(e_req + 1, S, (uint32_t)(e_req + 1), 0u);
      });
      const uint32_t old_x = x;
      x = xa1;
      xb = xb1;
      xa1 = xa2;
      xb1 = old_x;
    };
    super_stage(std::true_type{}, 0);
    {
      int s = 1;   // S >= 2: no guard in front of the loop
      do super_stage(std::false_type{}, s); while (++s < S);
    }

    // Every load in flight must have landed, in every wave, before the slots vacated last become the
    // staging area.  The s_nops are the wait states between the last MFMAs and the first reads of their
    // accumulators by other instructions.
    const int em0 = cur_tile.m0 + wm0, en0 = cur_tile.n0 + wn0;
    const int bz = cur_tile.bz;
    const int le = lane_id();
    constexpr bool LINEAR_BIAS = EPI == EPI_BIAS || EPI == EPI_BIAS_RELU || EPI == EPI_CLIPPED || EPI == EPI_SIGMOID ||
                                 EPI == EPI_TANH || EPI == EPI_ELU;
    u32x2_t bias_regs[8];
    if (LINEAR_BIAS) m16::load_bias<T, 4>(p, em0, en0, le, bias_regs);   // lands during the wait below
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier\n\ts_nop 7\n\ts_nop 7" ::: "memory");
    if (LINEAR_BIAS) m16::pin_all<4, 4>(acc);
    const int n_end = cur_tile.n0 + TILE;
    // staging: the slots of A_{S-1} (waves 0, 1) and B_{S-1} (waves 2, 3), half a slot each; x is A_S's by now
    uint32_t sa = x < lds + 2 * UNIT ? x + 3 * UNIT : x - 2 * UNIT;
    uint32_t sb = x < lds + UNIT ? x + 4 * UNIT : x - UNIT;
    const uint32_t stage = ((wave & 2) ? sb : sa) + (uint32_t)(wave & 1) * (uint32_t)(UNIT / 2);

    if (EPI == EPI_BIAS) m16::store_tile<T, 4, true, 0, false, 4>(p, acc, em0, en0, bz, le, stage, bias_regs, n_end);
    else if (EPI == EPI_RELU) m16::store_tile<T, 4, false, 1, false, 4>(p, acc, em0, en0, bz, le, stage, bias_regs, n_end);
    else if (EPI == EPI_BIAS_RELU) m16::store_tile<T, 4, true, 1, false, 4>(p, acc, em0, en0, bz, le, stage, bias_regs, n_end);
    else if (EPI == EPI_CLIPPED) m16::store_tile<T, 4, true, 2, false, 4>(p, acc, em0, en0, bz, le, stage, bias_regs, n_end);
    else if (EPI == EPI_SIGMOID) m16::store_tile<T, 4, true, 3, false, 4>(p, acc, em0, en0, bz, le, stage, bias_regs, n_end);
    else if (EPI == EPI_TANH) m16::store_tile<T, 4, true, 4, false, 4>(p, acc, em0, en0, bz, le, stage, bias_regs, n_end);
    else if (EPI == EPI_ELU) m16::store_tile<T, 4, true, 5, false, 4>(p, acc, em0, en0, bz, le, stage, bias_regs, n_end);
    else m16::store_tile<T, 4, false, 0, false, 4>(p, acc, em0, en0, bz, le, stage, bias_regs, n_end);
    if (!has_next) break;

    // every wave has finished reading its staging area before any wave's loads overwrite it
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    v = vn;
    cur_tile = next_tile;
  }
}

#undef SRT_FENCE

template <typename T, bool A_KC, bool B_KC, int EPI>
__global__ __launch_bounds__(NT) void gemm_m16q_kernel(GemmProblem p) {
  gemm_m16q_body<T, A_KC, B_KC, EPI>(p);
}

// ---- host side ---------------------------------------------------------------------------------------
template <typename T, bool A_KC, bool B_KC, int EPI>
hipError_t launch_kernel(const GemmProblem& p, hipStream_t stream) {
  auto kernel = gemm_m16q_kernel<T, A_KC, B_KC, EPI>;
  constexpr int lds_bytes = UNITS * UNIT;
  static std::atomic<uint32_t> configured{0};
  if (hipError_t e = ensure_lds_limit(reinterpret_cast<const void*>(kernel), lds_bytes, configured); e != hipSuccess) return e;
  const long long tiles = (long long)((p.M + TILE - 1) / TILE) * ((p.N + TILE - 1) / TILE) * p.batch;
  const int grid = ring::persistent_grid(tiles);
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(NT), lds_bytes, stream, p);
  return launch_status(stream);
}

template <typename T, bool A_KC, bool B_KC>
hipError_t launch(const GemmProblem& p, hipStream_t stream) {
  if (p.activation == srtActivationSigmoid) return launch_kernel<T, A_KC, B_KC, EPI_SIGMOID>(p, stream);
  if (p.activation == srtActivationTanh) return launch_kernel<T, A_KC, B_KC, EPI_TANH>(p, stream);
  if (p.activation == srtActivationElu) return launch_kernel<T, A_KC, B_KC, EPI_ELU>(p, stream);
  if (p.activation == srtActivationClippedRelu) return launch_kernel<T, A_KC, B_KC, EPI_CLIPPED>(p, stream);
  if (p.activation == srtActivationRelu) {
    if (p.bias) return launch_kernel<T, A_KC, B_KC, EPI_BIAS_RELU>(p, stream);
    return launch_kernel<T, A_KC, B_KC, EPI_RELU>(p, stream);
  }
  if (p.bias) return launch_kernel<T, A_KC, B_KC, EPI_BIAS>(p, stream);
  return launch_kernel<T, A_KC, B_KC, EPI_PLAIN>(p, stream);
}

}  // namespace m16q
}  // namespace srt
