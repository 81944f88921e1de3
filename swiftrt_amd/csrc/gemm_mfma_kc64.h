// 256 x 256 bf16 / fp16 matmul tile kernel for the layout where BOTH operands are stored
// k-contiguous (lhs not transposed, rhs transposed: y = x . W^T with W stored [N, K]).
//
// Why a second kernel for this layout: the ring kernel stages 32 k per row per stage, which for a
// k-contiguous row is half a 128-byte cache line -- with both operands stored that way every L2
// request is a half line, the request rate doubles and the matrix pipe starves (measured 72 %
// busy against 81 % for the other layouts).  Here a stage is 64 k deep, so every global load
// instruction moves whole lines (32 rows x 128 B per workgroup-wide instruction).  Two such stages
// fill 128 KiB of LDS, which leaves no room for a deep LDS ring; the prefetch distance comes from
// registers instead: the loads of stage P+2 are in flight in 64 VGPRs per lane while stage P is
// multiplied and stage P+1 sits in the other LDS slot.
//
//   LDS      2 slots x (A region 32 KiB + B region 32 KiB); a region is [256 rows][8 chunks of
//            16 B], chunk c of row r at position c ^ ((r >> 1) & 7): ds_write_b128 (lane = row
//            t / 8, chunk t % 8) and ds_read_b128 (lane = row l % 32, chunk 2 s + l / 32) are both
//            free of bank conflicts.
//   stage P  four k slices of 16 MFMAs per wave.  During slices 0 and 1 each lane writes its 16
//            registers of stage P+1 into the other slot and refills each register at once with
//            its load of stage P+2; the fragments of the next slice are read one slice ahead.
//            One barrier per stage, at the end of slice 2: by then every wave has read all of
//            stage P into registers (slot P is free for the writes of the next stage) and has
//            written its share of stage P+1 (visible to all for the reads that ride on slice 3).
//   epilogue the ring kernel's (same accumulator layout: C^T tiles, LDS-staged 16-byte stores).
#pragma once
#include "gemm_mfma_ring.h"

namespace srt {
namespace kc64 {

using namespace ring;

constexpr int KBK = 64;                      // k depth of a stage
constexpr int KREGION = 256 * KBK * 2;       // 32 KiB per operand
constexpr int KSLOT = 2 * KREGION;           // 64 KiB
#define SRT_FENCE() __builtin_amdgcn_sched_barrier(0)

__device__ __forceinline__ u32x4_t load_b128(__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff) {
  return __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)voff, (int)soff, 0);
}

template <typename T, int EPI>
__global__ __launch_bounds__(NT) void gemm_kc64_kernel(GemmProblem p) {
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
  const long long lda = p.sam, ldb = p.sbn;
  // bytes spanned by each operand view: anything beyond reads as zero (rows >= M / N start past it)
  const uint32_t a_bytes = (uint32_t)(((long long)(p.M - 1) * lda + p.K) * 2);
  const uint32_t b_bytes = (uint32_t)(((long long)(p.N - 1) * ldb + p.K) * 2);
  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(A), 0, (int)a_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(B), 0, (int)b_bytes, 0x00020000);

  // ---- global side: load i (0..7) of an operand covers tile rows 32 i + tid / 8, chunk tid % 8 ----
  const int lrow = tid >> 3, lchunk = tid & 7;
  uint32_t voa[8], vob[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    voa[i] = (uint32_t)(((long long)(m0 + 32 * i + lrow) * lda + lchunk * 8) * 2);
    vob[i] = (uint32_t)(((long long)(n0 + 32 * i + lrow) * ldb + lchunk * 8) * 2);
  }
  // ---- LDS write side: same (row, chunk), swizzled; load i lands 32 rows = 4 KiB further ----
  const uint32_t wr = (uint32_t)(lrow * 128 + ((lchunk ^ ((lrow >> 1) & 7)) << 4));
  // ---- LDS read side: fragment (tile t, slice s) = row 32 t + l % 32, chunk 2 s + l / 32 ----
  const int fr = lane & 31, fh = lane >> 5, ff = (fr >> 1) & 7;
  uint32_t rda[4], rdb[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const uint32_t c = (uint32_t)(((2 * s + fh) ^ ff) << 4);
    rda[s] = (uint32_t)((wm0 + fr) * 128) + c;
    rdb[s] = (uint32_t)(KREGION + (wn0 + fr) * 128) + c;
  }
  auto read_a = [&](uint32_t slot, int t, int s) {
    return *reinterpret_cast<const SRT_LDS u32x4_t*>(slot + rda[s] + t * 4096);
  };
  auto read_b = [&](uint32_t slot, int t, int s) {
    return *reinterpret_cast<const SRT_LDS u32x4_t*>(slot + rdb[s] + t * 4096);
  };

  f32x16_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  const int KT = (p.K + KBK - 1) / KBK;
  // first 16-byte chunk of the last stage that lies at or beyond K (8 = the stage is whole); K is a
  // multiple of 8, so chunks are never split
  const int tail_from = (p.K % KBK) ? (p.K % KBK) / 8 : 8;
  auto mask_tail = [&]() {   // aim this lane's chunk out of range for good (only the last stage is left)
    if (lchunk >= tail_from) {
#pragma unroll
      for (int i = 0; i < 8; ++i) voa[i] = vob[i] = OOB;
    }
  };
  auto soff_of = [&](int stage) { return stage < KT ? (uint32_t)stage * (KBK * 2) : OOB; };

  // ---- prologue: stage 0 through registers into slot 0, stage 1 into the registers ----
  u32x4_t ga[8], gb[8];
  if (tail_from < 8 && KT == 1) mask_tail();
  {
    const uint32_t so = soff_of(0);
    // same issue order as in the loop (all of A, then all of B), so the loop's waits are exact
#pragma unroll
    for (int i = 0; i < 8; ++i) ga[i] = load_b128(ra, voa[i], so);
#pragma unroll
    for (int i = 0; i < 8; ++i) gb[i] = load_b128(rb, vob[i], so);
#pragma unroll
    for (int i = 0; i < 8; ++i) *reinterpret_cast<SRT_LDS u32x4_t*>(lds + wr + i * 4096) = ga[i];
#pragma unroll
    for (int i = 0; i < 8; ++i) *reinterpret_cast<SRT_LDS u32x4_t*>(lds + KREGION + wr + i * 4096) = gb[i];
    if (tail_from < 8 && KT == 2) mask_tail();
    const uint32_t s1 = soff_of(1);
#pragma unroll
    for (int i = 0; i < 8; ++i) ga[i] = load_b128(ra, voa[i], s1);
#pragma unroll
    for (int i = 0; i < 8; ++i) gb[i] = load_b128(rb, vob[i], s1);
  }
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  SRT_FENCE();

  u32x4_t af[2][4], bf[2][4];   // [slice parity][32-wide tile]
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    af[0][t] = read_a(lds, t, 0);
    bf[0][t] = read_b(lds, t, 0);
  }

  uint32_t cur = lds, oth = lds + KSLOT;
  for (int kt = 0; kt < KT; ++kt) {
    // the loads issued in this trip are those of stage kt + 2
    if (tail_from < 8 && kt + 2 == KT - 1) mask_tail();
    const uint32_t so = soff_of(kt + 2);
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int par = s & 1;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int u = i * 4 + j;   // 0..15
          SRT_FENCE();
          acc[i][j] = mfma<T>(bf[par][j], af[par][i], acc[i][j]);
          SRT_FENCE();
          // fragments of the next slice (slice 0 of the next stage from the other slot), in the
          // order of their first use: a0 b0 b1 b2 b3 a1 a2 a3
          if (u < 8) {
            const uint32_t from = s < 3 ? cur : oth;
            const int ns = (s + 1) & 3;
            if (u == 0) af[par ^ 1][0] = read_a(from, 0, ns);
            else if (u <= 4) bf[par ^ 1][u - 1] = read_b(from, u - 1, ns);
            else af[par ^ 1][u - 4] = read_a(from, u - 4, ns);
          }
          // stage kt+1: registers -> other slot, then refill the register with stage kt+2
          if (s < 2 && (u & 1) == 0) {
            const int w = s * 8 + (u >> 1);   // 0..15: A loads 0..7, then B loads 0..7
            if (w < 8) {
              *reinterpret_cast<SRT_LDS u32x4_t*>(oth + wr + w * 4096) = ga[w];
              ga[w] = load_b128(ra, voa[w], so);
            } else {
              *reinterpret_cast<SRT_LDS u32x4_t*>(oth + KREGION + wr + (w - 8) * 4096) = gb[w - 8];
              gb[w - 8] = load_b128(rb, vob[w - 8], so);
            }
          }
        }
      }
      if (s == 2) {
        // every wave: all of stage kt is in registers or already multiplied, stage kt+1 is written
        SRT_FENCE();
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        SRT_FENCE();
      }
    }
    const uint32_t t = cur;
    cur = oth;
    oth = t;
  }
  // all LDS traffic of the main loop has retired in every wave before the slots become the
  // epilogue's staging area
  constexpr bool LINEAR_BIAS = EPI == EPI_BIAS || EPI == EPI_BIAS_RELU || EPI == EPI_CLIPPED;
  u32x2_t bias_regs[16];
  if (LINEAR_BIAS) load_bias<T>(p, m0 + wm0, n0 + wn0, lane, bias_regs);   // lands during the wait below
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  if (LINEAR_BIAS) pin_all(acc);   // no copy out of the accumulators is scheduled ahead of the wait
  const uint32_t stage = lds + (uint32_t)wave * 16384u;

  if (EPI == EPI_TRANS) {
    load_bias<T>(p, m0 + wm0, n0 + wn0, lane, bias_regs);   // one round of latency, before any store is in flight
    store_tile_transcendental<T>(p, acc, m0 + wm0, n0 + wn0, bz, lane, stage, bias_regs);
  } else {
    store_tile_linear<T, EPI>(p, acc, m0 + wm0, n0 + wn0, bz, lane, stage, bias_regs);
  }
}

#undef SRT_FENCE

// Same host-side preconditions as the ring kernel (32-bit byte offsets reach every view, C takes
// aligned 16-byte stores); both operands must be k-contiguous.
inline bool fits(const GemmProblem& p) { return ring_fits(p, true, true); }

template <typename T, int EPI>
hipError_t launch_kernel(const GemmProblem& p, hipStream_t stream) {
  auto kernel = gemm_kc64_kernel<T, EPI>;
  constexpr int lds_bytes = 2 * KSLOT;
  static std::atomic<uint32_t> configured{0};
  if (hipError_t e = ensure_lds_limit(reinterpret_cast<const void*>(kernel), lds_bytes, configured); e != hipSuccess) return e;
  const int tiles = ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
  hipLaunchKernelGGL(kernel, dim3(tiles, p.batch), dim3(NT), lds_bytes, stream, p);
  return launch_status(stream);
}

template <typename T>
hipError_t launch(const GemmProblem& p, hipStream_t stream) {
  const bool trans = p.activation == srtActivationSigmoid || p.activation == srtActivationTanh ||
                     p.activation == srtActivationElu;
  if (trans) return launch_kernel<T, EPI_TRANS>(p, stream);
  if (p.activation == srtActivationClippedRelu) return launch_kernel<T, EPI_CLIPPED>(p, stream);
  if (p.activation == srtActivationRelu) {
    if (p.bias) return launch_kernel<T, EPI_BIAS_RELU>(p, stream);
    return launch_kernel<T, EPI_RELU>(p, stream);
  }
  if (p.bias) return launch_kernel<T, EPI_BIAS>(p, stream);
  return launch_kernel<T, EPI_PLAIN>(p, stream);
}

}  // namespace kc64
}  // namespace srt
