// 128 x 128 fp32 matmul tile kernel for gfx950 on v_mfma_f32_32x32x2_f32 (true fp32 products and sums), built on
// the skeleton of the 16-bit quarter tile (gemm_mfma_m16q.h): direct-to-LDS loads of whole cache lines into a ring
// of five 32 KiB slots, requests two super-stages ahead, one barrier per super-stage, a persistent XCD-aware tile
// walk that runs on across tile boundaries, MFMAs written out with the accumulators tied.
//
// An fp32 MFMA holds the matrix pipe four times as long per byte of operand as a bf16 one does, so everything but
// the MFMAs is cheap here and the point of the design is only that nothing ever makes the pipe wait: the register-
// staged 128 x 128 kernel of gemm_f32.hip (a barrier pair and a round trip global -> registers -> LDS per 16 k, hidden
// only by co-resident workgroups) reaches 0.75 of the fp32 matrix rate at four workgroups per unit and 0.58 at one.
//
// Tile: 128 x 128 per workgroup, four waves 2 x 2, a wave 64 x 64 = 2 x 2 MFMA tiles of 32 x 32 (64 accumulator
// registers).  A unit of staging is one operand, 128 rows (columns) x 64 k = 32 KiB; a super-stage is 64 k = eight
// octets of 8 k, 16 MFMAs each (four k pairs x 2 x 2 tiles), 128 MFMAs = 8192 cycles per wave.
// Layouts of a unit:
//   k-contiguous operand:  [128 rows][16 chunks of 16 B = 4 k], chunk c of row r at position c ^ (r & 15).  Lane l
//                          (row l % 32, half h = l / 32) takes chunk 2 o + h of octet o with one ds_read_b128: its four
//                          values are k = 8 o + 4 h + 0..3, and MFMA m of the octet multiplies component m -- the k
//                          pair (8 o + m, 8 o + 4 + m).
//   mn-contiguous operand: [64 k][32 chunks of 16 B = 4 m], chunk c of k row k at c ^ (((k >> 2) & 1) << 3) (the two
//                          half waves read k rows four apart: the swizzle puts them on different banks).  The same
//                          four values come from four ds_read_b32 at k rows 8 o + 4 h + 0..3.
// A load instruction moves 1 KiB: 4 rows x 256 B (k-contiguous) or 2 k rows x 512 B; a wave issues eight per unit.
// Schedule of super-stage s (octets 0-7; fragment set = octet mod 2; the four fragments of the next octet are read
// into the idle set behind MFMAs 0, 4, 8, 12):
//   octet 0      scalar bookkeeping for the request of A_{s+2}
//   octets 1, 2  the eight loads of A_{s+2} (into the slot of B_{s-1})
//   octets 3-6   --
//   sync         s_waitcnt vmcnt(8) lgkmcnt(0); s_barrier (after octet 6, whose reads are the unit's last)
//   octet 7      the eight loads of B_{s+2} (into the slot of A_s); reads octet 0 of super-stage s + 1
// Preconditions (f32_ring_fits): both operands contiguous along k or along m / n with 16-byte aligned rows, K a
// multiple of 64 and at least 128, the result's columns contiguous, 32-bit byte offsets reach every operand.
#pragma once
#include "gemm_mfma_ring.h"

namespace srt {
namespace f32r {

using ring::NT;
using ring::OOB;
using ring::u32x4_t;

typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4v_t __attribute__((ext_vector_type(4)));

constexpr int DK = 64;               // k depth of a unit
constexpr int UNIT = 128 * DK * 4;  // a slot of the ring: 32 KiB, the unit of 128 rows (one of 64 rows fills half)
constexpr int UNITS = 5;

#define SRT_FENCE() __builtin_amdgcn_sched_barrier(0)

__device__ __forceinline__ uint32_t select_lt(int a, int b, uint32_t t, uint32_t f) {
  uint32_t r;
  asm("s_cmp_lt_i32 %1, %2\n\ts_cselect_b32 %0, %3, %4" : "=s"(r) : "s"(a), "s"(b), "s"(t), "s"(f) : "scc");
  return r;
}

// acc += a x b: a supplies rows, b columns; lane l of the result holds column l % 32 and rows 8 (v / 4) + 4 (l / 32) + v % 4.
// (Held transposed -- B's fragment first, so that a lane owns one row and runs of four consecutive columns and stores 16
// bytes at a time -- the epilogue is slower: an instruction then touches 32 rows with 32 bytes each, where this way a half
// wave writes one whole 128-byte line; 4096^3 997 us against 969, 8192 x 8192 x 1024 1186 against 1086.)
__device__ __forceinline__ void mfma32(f32x16_t& acc, float a, float b) {
  asm volatile("v_mfma_f32_32x32x2_f32 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma32_first(f32x16_t& acc, float a, float b) {
  asm volatile("v_mfma_f32_32x32x2_f32 %0, %1, %2, 0" : "=a"(acc) : "v"(a), "v"(b));
}

// ---- global -> LDS.  A unit holds ROWS = 128 or 64 rows (columns) of an operand; a wave issues ROWS / 16 loads per
// unit; load i takes lane offset voff[i & 3], scalar offset so[i >> 2], and lands at the wave's share + i KiB ----
template <bool KC, int ROWS>
struct Loader {
  static constexpr int LOADS = ROWS / 16;
  uint32_t voff[4];
  static __device__ __forceinline__ uint32_t wave_share(int wave) { return (uint32_t)wave * (uint32_t)(ROWS * 64); }
  // bytes between so[0] and so[1] (ROWS = 128 only): 16 rows (KC) or 8 k rows (MN)
  static __device__ __forceinline__ uint32_t step(long long ld) { return (uint32_t)((KC ? 16 : 8) * ld * 4); }

  // ld: elements between rows (KC: rows are m or n; MN: rows are k)
  __device__ __forceinline__ void init(int wave, int lane, long long ld) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (KC) {
        // a load: 4 rows x 256 B; the wave's rows: ROWS / 4 (loads 4-7 of 128 rows: + 16, which the swizzle does not see)
        const int row = wave * (ROWS / 4) + i * 4 + (lane >> 4);
        const int chunk = (lane & 15) ^ (row & 15);
        voff[i] = (uint32_t)(((long long)row * ld + chunk * 4) * 4);
      } else if constexpr (ROWS == 128) {
        const int krow = wave * 16 + i * 2 + (lane >> 5);   // a load: 2 k rows x 512 B; + 8 for loads 4-7: bit 2 of k is untouched
        const int chunk = (lane & 31) ^ (((krow >> 2) & 1) << 3);
        voff[i] = (uint32_t)(((long long)krow * ld + chunk * 4) * 4);
      } else {
        const int krow = wave * 16 + i * 4 + (lane >> 4);   // a load: 4 k rows x 256 B
        const int chunk = (lane & 15) ^ (((krow >> 2) & 1) << 3);
        voff[i] = (uint32_t)(((long long)krow * ld + chunk * 4) * 4);
      }
    }
  }
};

// ---- LDS -> MFMA operands: the four values k = 8 o + 4 h + 0..3 of row (column) row0 + 32 t + l % 32 ----
template <bool KC, int ROWS>
struct FragReader;
template <int ROWS>
struct FragReader<true, ROWS> {
  uint32_t off[2];   // octet parity: chunk 2 o + h = (2 (o & 1) + h) + 4 (o >> 1); tile t adds t * 8192
  __device__ __forceinline__ void init(int lane, int row0) {
    const int r = lane & 31, h = lane >> 5;
    const int row = row0 + r;   // row0 is a multiple of 32: row & 15 = r & 15, also for tile 1
#pragma unroll
    for (int p = 0; p < 2; ++p) off[p] = (uint32_t)(row * 256 + (((2 * p + h) ^ (r & 15)) << 4));
  }
  template <int O>
  __device__ __forceinline__ f32x4v_t read(uint32_t unit, int t) const {
    // chunk 2 O + h: bits 2-3 of the chunk index are O >> 1, and the swizzle is an XOR
    return *reinterpret_cast<const SRT_LDS f32x4v_t*>(unit + (off[O & 1] ^ (uint32_t)((O >> 1) << 6)) + t * 8192);
  }
};
template <int ROWS>
struct FragReader<false, ROWS> {
  static constexpr int PITCH = ROWS * 4;   // bytes per k row
  uint32_t off[2];   // per tile (the swizzle depends on h only: k rows 8 o + 4 h + m have bit 2 = h)
  __device__ __forceinline__ void init(int lane, int row0) {
    const int r = lane & 31, h = lane >> 5;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int mn = (row0 + 32 * t + r) & (ROWS - 1);   // (tile 1 of a one-tile wave is never read)
      off[t] = (uint32_t)((4 * h) * PITCH + ((((mn >> 2) ^ (h << 3)) << 4) | ((mn & 3) << 2)));
    }
  }
  template <int O>
  __device__ __forceinline__ f32x4v_t read(uint32_t unit, int t) const {
    const uint32_t a = unit + off[t] + O * 8 * PITCH;   // 8 k rows per octet
    f32x4v_t v;
    v[0] = *reinterpret_cast<const SRT_LDS float*>(a);
    v[1] = *reinterpret_cast<const SRT_LDS float*>(a + PITCH);
    v[2] = *reinterpret_cast<const SRT_LDS float*>(a + 2 * PITCH);
    v[3] = *reinterpret_cast<const SRT_LDS float*>(a + 3 * PITCH);
    return v;
  }
};

struct TileAt {
  uint32_t offa, offb;
  int m0, n0, bz;
};

// ---- accumulators -> result.  Lane l of accumulator tile (i, j) holds column 32 j + l % 32 and rows
// 32 i + 8 (q / 4) + 4 (l / 32) + q % 4, q = 0..15. ----
// The activation fixed at compile time, BIAS: a bias per column (both values a lane needs are fetched before the first
// store: a wait on a load is a wait on everything in flight, the next tile's requests included, so there is one per
// tile and none without a bias); INTERIOR: the tile lies inside the result.
// (acc + 0 where there is no bias, as the general form has it: the same bits whatever the path.)
template <int ACT, bool BIAS, bool INTERIOR, int TM, int TN>
__device__ __forceinline__ void store_tile(const GemmProblem& p, const TileAt& t, f32x16_t (&acc)[TM][TN], int wm0, int wn0, int lane) {
  const int r = lane & 31, h = lane >> 5;
  float* C = (float*)p.C + (long long)t.bz * p.scb;
  float b[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) b[j] = 0.0f;
  if constexpr (BIAS) {
    const float* bias = (const float*)p.bias;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = t.n0 + wn0 + 32 * j + r;
      if (INTERIOR || n < p.N) b[j] = bias[(long long)n * p.sbias];
    }
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = t.n0 + wn0 + 32 * j + r;
      const int mb = t.m0 + wm0 + 32 * i + 4 * h;
      const bool n_in = INTERIOR || n < p.N;
      float* c = C + (long long)mb * p.scm + (long long)n * p.scn;
      asm volatile("" : "+a"(acc[i][j]));
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const int mo = 8 * (q >> 2) + (q & 3);
        if (INTERIOR || (n_in && mb + mo < p.M)) c[(long long)mo * p.scm] = activation_ct<ACT>(p.coef, acc[i][j][q] + b[j]);
      }
    }
  }
}
template <int ACT, int TM, int TN>
__device__ __forceinline__ void store_tile_for(const GemmProblem& p, const TileAt& t, f32x16_t (&acc)[TM][TN], int wm0, int wn0, int lane) {
  const bool interior = t.m0 + 64 * TM <= p.M && t.n0 + 64 * TN <= p.N;
  if (p.bias) {
    if (interior) store_tile<ACT, true, true, TM, TN>(p, t, acc, wm0, wn0, lane);
    else store_tile<ACT, true, false, TM, TN>(p, t, acc, wm0, wn0, lane);
  } else {
    if (interior) store_tile<ACT, false, true, TM, TN>(p, t, acc, wm0, wn0, lane);
    else store_tile<ACT, false, false, TM, TN>(p, t, acc, wm0, wn0, lane);
  }
}
// Any epilogue of the interface (the activation switched per element).
template <int TM, int TN>
__device__ __forceinline__ void store_tile_any(const GemmProblem& p, const TileAt& t, f32x16_t (&acc)[TM][TN], int wm0, int wn0, int lane) {
  const int r = lane & 31, h = lane >> 5;
  float* C = (float*)p.C + (long long)t.bz * p.scb;
  Epilogue<F32> ep(p);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = t.n0 + wn0 + 32 * j + r;
      const int mb = t.m0 + wm0 + 32 * i + 4 * h;
      asm volatile("" : "+a"(acc[i][j]));
      float out[16];
#pragma unroll
      for (int q = 0; q < 16; ++q) out[q] = acc[i][j][q];
      ep.finish_run(out, [&](int q, int* m, int* nn) {
        *m = mb + 8 * (q >> 2) + (q & 3);
        *nn = n;
        return *m < p.M && n < p.N;
      });
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const int m = mb + 8 * (q >> 2) + (q & 3);
        if (m < p.M && n < p.N) C[(long long)m * p.scm + (long long)n * p.scn] = out[q];
      }
    }
  }
}

template <bool A_KC, bool B_KC, int TM, int TN>
__device__ __forceinline__ void gemm_f32_ring_body(const GemmProblem& p) {
  constexpr int ROWS_A = 64 * TM, ROWS_B = 64 * TN;   // the workgroup's tile
  constexpr int NA = ROWS_A / 16, NB = ROWS_B / 16;   // loads per wave and unit
  constexpr int NMO = 4 * TM * TN;                    // MFMAs per octet
  using LoaderA = Loader<A_KC, ROWS_A>;
  using LoaderB = Loader<B_KC, ROWS_B>;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[];
  const uint32_t lds = (uint32_t)(uintptr_t)(SRT_LDS unsigned char*)lds_raw;
  const uint32_t lds_end = lds + UNITS * UNIT;

  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  auto lane_id = []() {
    uint32_t zero = 0;
    asm volatile("" : "+s"(zero));
    return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, zero));
  };
  const int wm0 = (wave >> 1) * 32 * TM, wn0 = (wave & 1) * 32 * TN;

  const int tiles_m = (p.M + ROWS_A - 1) / ROWS_A, tiles_n = (p.N + ROWS_B - 1) / ROWS_B;
  const int total = tiles_m * tiles_n * p.batch;
  const int grid = (int)gridDim.x;
  int v = (int)blockIdx.x;
  if (v >= total) return;

  const long long lda = A_KC ? p.sam : p.sak;
  const long long ldb = B_KC ? p.sbn : p.sbk;
  const long long a_view = A_KC ? (long long)(p.M - 1) * lda + p.K : (long long)(p.K - 1) * lda + p.M;
  const long long b_view = B_KC ? (long long)(p.N - 1) * ldb + p.K : (long long)(p.K - 1) * ldb + p.N;
  const u32x4_t ra = ring::make_rsrc(p.A, (uint32_t)(((long long)(p.batch - 1) * p.sab + a_view) * 4));
  const u32x4_t rb = ring::make_rsrc(p.B, (uint32_t)(((long long)(p.batch - 1) * p.sbb + b_view) * 4));
  auto locate = [&](int tile) {
    const int per_batch = tiles_m * tiles_n;
    const int bz = tile / per_batch;
    int tm, tn;
    ring::tile_coords(tile - bz * per_batch, tiles_m, tiles_n, &tm, &tn);
    TileAt t;
    t.m0 = tm * ROWS_A;
    t.n0 = tn * ROWS_B;
    t.bz = bz;
    t.offa = (uint32_t)(((long long)bz * p.sab + (A_KC ? (long long)t.m0 * lda : (long long)t.m0)) * 4);
    t.offb = (uint32_t)(((long long)bz * p.sbb + (B_KC ? (long long)t.n0 * ldb : (long long)t.n0)) * 4);
    return t;
  };
  const uint32_t kstep_a = A_KC ? (uint32_t)(DK * 4) : (uint32_t)(DK * lda * 4);   // bytes per super-stage
  const uint32_t kstep_b = B_KC ? (uint32_t)(DK * 4) : (uint32_t)(DK * ldb * 4);
  const uint32_t lstep_a = LoaderA::step(lda), lstep_b = LoaderB::step(ldb);
  const int S = p.K / DK;   // super-stages per tile (whole ones, at least two)
  auto wrap = [&](uint32_t a) { return a >= lds_end ? a - UNITS * UNIT : a; };

  TileAt cur_tile = locate(v);

  auto issue_a = [&](const LoaderA& l, uint32_t slot, uint32_t base) {
#pragma unroll
    for (int i = 0; i < NA; ++i)
      ring::load_to_lds(ra, slot + LoaderA::wave_share(wave) + (uint32_t)i * 1024u, l.voff[i & 3],
                        base + (uint32_t)(i >> 2) * lstep_a);
  };
  auto issue_b = [&](const LoaderB& l, uint32_t slot, uint32_t base) {
#pragma unroll
    for (int i = 0; i < NB; ++i)
      ring::load_to_lds(rb, slot + LoaderB::wave_share(wave) + (uint32_t)i * 1024u, l.voff[i & 3],
                        base + (uint32_t)(i >> 2) * lstep_b);
  };

  uint32_t x = lds;   // slot of A_s; B_s follows it, then A_{s+1}, B_{s+1}, A_{s+2} (B_{s+2} goes where A_s is)

  bool first_tile = true;
  for (;;) {
    LoaderA la;
    LoaderB lb;
    FragReader<A_KC, ROWS_A> fa;
    FragReader<B_KC, ROWS_B> fb;
    const int lane = lane_id();
    la.init(wave, lane, lda);
    lb.init(wave, lane, ldb);
    fa.init(lane, wm0);
    fb.init(lane, wn0);
    uint32_t xb = wrap(x + UNIT), xa1 = wrap(x + 2 * UNIT), xb1 = wrap(x + 3 * UNIT);
    if (first_tile) {
      issue_a(la, x, cur_tile.offa);
      issue_b(lb, xb, cur_tile.offb);
      issue_a(la, xa1, cur_tile.offa + kstep_a);
      issue_b(lb, xb1, cur_tile.offb + kstep_b);
      if constexpr (NA + NB == 16) asm volatile("s_waitcnt vmcnt(16)\n\ts_barrier" ::: "memory");
      else if constexpr (NA + NB == 12) asm volatile("s_waitcnt vmcnt(12)\n\ts_barrier" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(8)\n\ts_barrier" ::: "memory");
    }   // (later tiles: their first two super-stages were requested during the previous tile)
    first_tile = false;
    SRT_FENCE();

    const int vn = v + grid;
    const bool has_next = vn < total;
    const TileAt next_tile = locate((int)select_lt(vn, total, (uint32_t)vn, (uint32_t)v));
    // requests below the limit are real: those of this tile and the first two super-stages of the next
    const int limit = (int)select_lt(vn, total, (uint32_t)(S + 2), (uint32_t)S);

    f32x16_t acc[TM][TN];   // defined by the MFMAs of the tile's first k pair
    f32x4v_t af[2][TM], bf[2][TN];   // [fragment set][tile]
#pragma unroll
    for (int t = 0; t < TM; ++t) af[0][t] = fa.template read<0>(x, t);
#pragma unroll
    for (int t = 0; t < TN; ++t) bf[0][t] = fb.template read<0>(xb, t);

    int e_req = S > 2 ? 2 : 0;   // k index of request s + 2
    uint32_t ea_off = (uint32_t)e_req * kstep_a, eb_off = (uint32_t)e_req * kstep_b;

    auto set_target = [](auto imm_tag, uint32_t base) __attribute__((always_inline)) {
      ring::set_lds_target<decltype(imm_tag)::value>(base);
    };

    // One octet: NMO MFMAs (u = TM TN m + TN i + j: k pair m, tile (i, j)) on fragment set CUR; the TM + TN fragments
    // of octet NO of the units (ua, ub) are read into the other set, spread over the octet in the order of first use.
    //   LOADS 0: none; 1: A loads 0-3; 2: A loads 4-7 (128 rows only); 3: all B loads (`target`: the request's slot plus
    //   the wave's share, so0 / so1: its scalar offsets), at most one per MFMA: the landing address goes into M0
    //   before the MFMA, the load follows it.  `ev(e)`, e = 0..15: scalar bookkeeping, 16 / NMO steps behind each MFMA.
    auto octet = [&](auto cur_tag, auto first_tag, auto no_tag, auto loads_tag, uint32_t ua, uint32_t ub,
                     const uint32_t& target, const uint32_t& so0, const uint32_t& so1, auto&& ev) __attribute__((always_inline)) {
      constexpr int CUR = decltype(cur_tag)::value, NXT = CUR ^ 1;
      constexpr bool FIRST = decltype(first_tag)::value;
      constexpr int NO = decltype(no_tag)::value;
      constexpr int LOADS = decltype(loads_tag)::value;
      constexpr int COUNT = LOADS == 3 ? NB : LOADS == 1 ? 4 : (LOADS == 2 && NA == 8) ? 4 : 0;
      constexpr int STRIDE = NMO / (COUNT > 0 ? COUNT : NMO);
      constexpr int READ_STRIDE = NMO / (TM + TN);
#pragma unroll
      for (int m = 0; m < 4; ++m) {
#pragma unroll
        for (int ij = 0; ij < TM * TN; ++ij) {
          const int i = ij / TN, j = ij % TN;
          const int u = TM * TN * m + ij;
          int ld = -1;
          if (COUNT && u % STRIDE == (STRIDE > 1 ? 1 : 0)) ld = u / STRIDE + (LOADS == 2 ? 4 : 0);
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
          if (FIRST && m == 0) mfma32_first(acc[i][j], af[CUR][i][m], bf[CUR][j][m]);
          else mfma32(acc[i][j], af[CUR][i][m], bf[CUR][j][m]);
          if (ld >= 0) {
            SRT_FENCE();
            const uint32_t so = (ld >> 2) == 0 ? so0 : so1;
            if (LOADS == 3) ring::load_to_lds_at_m0(rb, lb.voff[ld & 3], so);
            else ring::load_to_lds_at_m0(ra, la.voff[ld & 3], so);
          }
          if (u % READ_STRIDE == 0 && u / READ_STRIDE < TM + TN) {
            const int f = u / READ_STRIDE;   // a0 b0 (a1) (b1): the order of first use
            if (f == 0) af[NXT][0] = fa.template read<NO>(ua, 0);
            if (f == 1) bf[NXT][0] = fb.template read<NO>(ub, 0);
            if (TM == 2 && f == 2) af[NXT][TM - 1] = fa.template read<NO>(ua, TM - 1);
            if (TN == 2 && f == TM + 1) bf[NXT][TN - 1] = fb.template read<NO>(ub, TN - 1);
          }
#pragma unroll
          for (int e = u * (16 / NMO); e < (u + 1) * (16 / NMO); ++e) ev(e);
          SRT_FENCE();
        }
      }
    };

    using C0 = std::integral_constant<int, 0>;
    using C1 = std::integral_constant<int, 1>;
    using C2 = std::integral_constant<int, 2>;
    using C3 = std::integral_constant<int, 3>;
    using C4 = std::integral_constant<int, 4>;
    using C5 = std::integral_constant<int, 5>;
    using C6 = std::integral_constant<int, 6>;
    using C7 = std::integral_constant<int, 7>;
    using NO_FIRST = std::false_type;
    auto nothing = [](int) __attribute__((always_inline)) {};
    auto super_stage = [&](auto first_tag, int s) __attribute__((always_inline)) {
      const int r = s + 2;   // index of the units requested in this super-stage
      uint32_t xa2 = 0, sel = 0, soa = 0, sob = 0, ta = 0, tb = 0;
      uint32_t so_a0 = OOB, so_a1 = OOB, so_b0 = OOB, so_b1 = OOB;
      // ---- octet 0: the request of A_{s+2} is worked out ----
      octet(C0{}, first_tag, C1{}, C0{}, x, xb, ta, so_a0, so_a1, [&](int e) __attribute__((always_inline)) {
        if (e == 1) xa2 = xa1 + 2 * UNIT;
        if (e == 3) xa2 = select_lt((int)xa2, (int)lds_end, xa2, xa2 - UNITS * UNIT);
        if (e == 5) sel = select_lt(r, S, cur_tile.offa, next_tile.offa);
        if (e == 7) soa = select_lt(r, limit, sel + ea_off, OOB);
        if (e == 9) ta = xa2 + LoaderA::wave_share(wave);
        if (e == 11) so_a0 = soa;
        if (e == 13) so_a1 = select_lt(r, limit, soa + lstep_a, OOB);
      });
      // ---- octets 1, 2: the loads of A_{s+2}; the request of B_{s+2} is worked out ----
      octet(C1{}, NO_FIRST{}, C2{}, C1{}, x, xb, ta, so_a0, so_a1, [&](int e) __attribute__((always_inline)) {
        if (e == 3) sel = select_lt(r, S, cur_tile.offb, next_tile.offb);
        if (e == 7) sob = select_lt(r, limit, sel + eb_off, OOB);
      });
      octet(C0{}, NO_FIRST{}, C3{}, C2{}, x, xb, ta, so_a0, so_a1, [&](int e) __attribute__((always_inline)) {
        if (e == 3) so_b0 = sob;
        if (e == 7) so_b1 = select_lt(r, limit, sob + lstep_b, OOB);
        if (e == 11) tb = x + LoaderB::wave_share(wave);
      });
      // ---- octets 3-6 ----
      octet(C1{}, NO_FIRST{}, C4{}, C0{}, x, xb, ta, so_a0, so_a1, nothing);
      octet(C0{}, NO_FIRST{}, C5{}, C0{}, x, xb, ta, so_a0, so_a1, nothing);
      octet(C1{}, NO_FIRST{}, C6{}, C0{}, x, xb, ta, so_a0, so_a1, nothing);
      octet(C0{}, NO_FIRST{}, C7{}, C0{}, x, xb, ta, so_a0, so_a1, nothing);
      // ---- sync: all of super-stage s is in registers, A_{s+1} and B_{s+1} have landed (all but the newest
      // request's loads, those of A_{s+2}) ----
      if constexpr (NA == 8) asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      SRT_FENCE();
      // ---- octet 7: the loads of B_{s+2}; reads of super-stage s + 1 ----
      octet(C1{}, NO_FIRST{}, C0{}, C3{}, xa1, xb1, tb, so_b0, so_b1, [&](int e) __attribute__((always_inline)) {
        // the next request's k index: one further, or back to 0 past the tile's last super-stage
        if (e == 2) ea_off = select_lt(e_req + 1, S, ea_off + kstep_a, 0u);
        if (e == 6) eb_off = select_lt(e_req + 1, S, eb_off + kstep_b, 0u);
        if (e == 10) e_req = (int)select_lt(e_req + 1, S, (uint32_t)(e_req + 1), 0u);
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

    // ---- tile boundary: nothing to wait for.  The next tile's first two super-stages are requested (A'_0, B'_0 landed
    // and seen by every wave at the last sync; A'_1, B'_1 in flight into slots nobody reads any more), and the slot the
    // next request goes to was last read before that sync.  The stores count in vmcnt with the loads: the next sync
    // waits for "all but the newest NA", which the loads, returning in order, satisfy no later than before. ----
    asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory");   // the last MFMA's 16 passes, before its registers are read
    // ---- epilogue: straight from the accumulators (a half wave stores 128 contiguous bytes of a row), specialised
    // once per tile for the common epilogues: a tile is up to 64 stores per lane with nothing to overlap them ----
    {
      const int le = lane_id();
      const bool plain_bias = !p.bias || !p.bias_per_row;
      if (plain_bias && p.activation == srtActivationIdentity) store_tile_for<srtActivationIdentity, TM, TN>(p, cur_tile, acc, wm0, wn0, le);
      else if (plain_bias && p.activation == srtActivationRelu) store_tile_for<srtActivationRelu, TM, TN>(p, cur_tile, acc, wm0, wn0, le);
      else store_tile_any<TM, TN>(p, cur_tile, acc, wm0, wn0, le);
    }
    if (!has_next) break;
    v = vn;
    cur_tile = next_tile;
  }
}

#undef SRT_FENCE

template <bool A_KC, bool B_KC, int TM, int TN>
__global__ __launch_bounds__(NT) void gemm_f32_ring_kernel(GemmProblem p) {
  gemm_f32_ring_body<A_KC, B_KC, TM, TN>(p);
}

}  // namespace f32r
}  // namespace srt
