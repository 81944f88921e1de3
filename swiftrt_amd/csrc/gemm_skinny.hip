// Small-M matmul (M <= 64) against a k-contiguous weight: out[m, n] = sum_k x[m, k] * W[n, k].
// The shape of single-token / small-batch inference; bound by streaming W from HBM once.
//
//   block   4 waves share 32 rows of W (one 32 x 32 output tile; rows m >= M are zero).  Wave w
//           takes the 64-wide k blocks w, w + 4, ...; the four partial tiles are summed through
//           LDS once at the end, then bias + activation + store.
//   W       streams HBM -> LDS with `buffer_load_dwordx4 ... lds`, fully coalesced: one load
//           instruction fetches 8 rows x 128 contiguous bytes (whole cache lines), four per k
//           block.  Each wave owns a private ring of DEPTH k blocks in LDS (no workgroup barrier
//           in the k loop, only s_waitcnt on the wave's own loads), so DEPTH (2-3) x 4 KiB per wave
//           are in flight at any time.  LDS layout per block: [32 rows][8 chunks of 16 B], chunk c
//           of row r at c ^ ((r >> 1) & 7): the MFMA B-operand read (lane l: row l % 32, chunk
//           2 s + l / 32) is one conflict-free ds_read_b128.
//   x       is tiny and hits in L2; its rows for the same k block ride in the same ring slot
//           (8, 16 or 32 staged rows, one load instruction per 8), so the k loop's only
//           vector-memory instructions are global->LDS loads and its only register-producing
//           loads are LDS reads.
//   grid    ceil(N / 32) x batch workgroups of 60-72 KiB LDS: two per CU, all resident at once.
//   W[K,N]  An n-contiguous weight (x . W, the Dense layer's own layout) streams the same way with 64
//           columns per workgroup: a k row of the block is then 128 contiguous bytes, one load
//           instruction fetches 8 k rows, and a k block of 64 rows lands as [64 k][8 chunks of 16 B],
//           chunk c of k row k at c ^ (((k >> 1) & 1) << 2).  The MFMA operand (lane l: column l % 32,
//           k = 8 (l / 32) .. + 7) is two ds_read_b64_tr_b16: within 16 lanes the instruction
//           transposes a 4 (k) x 16 (n) block; the swizzle puts the four k rows a half wave touches
//           on different banks.
//   M > 32  two 32-row output tiles per 32 rows of W (the x fragments of both meet each W fragment)
//   M > 16  x is as large per k block as the 32 rows of W it meets, and every workgroup re-reads it
//           from L2: when N is large enough to keep most CUs busy that way, a workgroup takes 64
//           rows of W (two output tiles per wave sharing the x fragments): 12 loads per k block and
//           64 columns instead of 16, x traffic halved.
#include "gemm_common.h"

namespace srt {

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
#define SRT_LDS __attribute__((address_space(3)))

template <typename T>
__device__ __forceinline__ f32x16_t mfma32s(u32x4_t a, u32x4_t b, f32x16_t c);
template <>
__device__ __forceinline__ f32x16_t mfma32s<BF16>(u32x4_t a, u32x4_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b),
                                                 c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x16_t mfma32s<F16>(u32x4_t a, u32x4_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b),
                                                c, 0, 0, 0);
}

// fp32: a 16-byte fragment holds four k values; component m of both operands is the k pair (8 s + m, 8 s + 4 + m) of the
// two half waves, and the four pairs take four v_mfma_f32_32x32x2_f32.
template <>
__device__ __forceinline__ f32x16_t mfma32s<F32>(u32x4_t a, u32x4_t b, f32x16_t c) {
  typedef float f32x4_t __attribute__((ext_vector_type(4)));
  const f32x4_t af = __builtin_bit_cast(f32x4_t, a), bf = __builtin_bit_cast(f32x4_t, b);
  c = __builtin_amdgcn_mfma_f32_32x32x2f32(af.x, bf.x, c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_32x32x2f32(af.y, bf.y, c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_32x32x2f32(af.z, bf.z, c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_32x32x2f32(af.w, bf.w, c, 0, 0, 0);
  return c;
}

constexpr int SK_WAVES = 4;
constexpr int SK_WTILE = 32 * 128;    // one 32-row W tile of a ring slot: 32 rows x 128 B
constexpr uint32_t SK_OOB = 0x80000000u;

// XR: x rows staged per k block; NW: 32-row W tiles per workgroup.  Ring depth: what fits in
// 160 KiB of LDS with two workgroups per CU (NW = 1) or one (NW = 2).
template <int XR, int NW>
struct SkinnyShape {
  static constexpr int MT = (XR + 31) / 32;                          // 32-row output tiles along M
  static constexpr int DEPTH = XR == 64 ? (NW == 2 ? 2 : 3) : NW == 2 ? 3 : (XR == 32 ? 2 : 3);   // k blocks in flight per wave
  static constexpr int WBYTES = NW * SK_WTILE;                      // W part of a ring slot
  static constexpr int SLOT = WBYTES + XR * 128;                    // W rows + x rows of one k block
  static constexpr int LOADS = 4 * NW + XR / 8;                     // load instructions per k block
  static constexpr int LDS = SK_WAVES * DEPTH * SLOT;               // 60 / 72 / 64 KiB; 128-144 KiB for NW = 2 or XR = 64
};

// STREAM: the data is read once by the whole grid (the weight), so the load carries the
// non-temporal hint and its lines do not linger in L2 -- measured on a bare streaming loop of
// this access pattern: 5.7 TB/s without the hint, 6.1-6.2 TB/s with it.  x, which every
// workgroup re-reads, keeps the default policy.
template <bool STREAM>
__device__ __forceinline__ void sk_load_to_lds(u32x4_t rsrc, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
  if (STREAM) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen nt lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
                 : "memory");
  } else {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
                 : "memory");
  }
}

// XR = number of x rows staged per k block (8, 16, 32 or 64 >= M).
// Every vector-memory instruction in the k loop is a global->LDS load issued from inline assembly
// and awaited with explicit s_waitcnt vmcnt; everything that produces registers is an LDS read,
// which the compiler tracks on its own counter.
// W_MN: the weight is n-contiguous ([K, N]); a workgroup takes 32 NW columns, i.e. RB = 64 NW bytes
// of every k row.
template <typename T, int XR, int NW, bool W_MN = false>
__global__ __launch_bounds__(SK_WAVES * 64) void gemm_skinny_kernel(GemmProblem p) {
  constexpr int ES = (int)sizeof(typename T::storage);   // element size
  constexpr int EPC = 16 / ES;                           // elements per 16-byte chunk
  constexpr int KBE = 128 / ES;                          // k per block
  constexpr int RB = 32 * NW * ES;   // W_MN: bytes of a k row in LDS (the workgroup's 32 NW columns)
  static_assert(ES == 2 || !W_MN || NW == 1, "fp32 against an n-contiguous weight: one tile of 32 columns = whole 128-byte lines");
  using Shape = SkinnyShape<XR, NW>;
  constexpr int SK_WBYTES = Shape::WBYTES;
  constexpr int MT = Shape::MT;
  constexpr int DEPTH = Shape::DEPTH;
  extern __shared__ __attribute__((aligned(1024))) unsigned char sk_lds_raw[];
  const uint32_t lds = (uint32_t)(uintptr_t)(SRT_LDS unsigned char*)sk_lds_raw;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, h = lane >> 5;
  // columns of this workgroup: 32 NW, or fewer (a multiple of 8) when the launcher narrowed the tile so that
  // the workgroups come out even over the compute units; what lies beyond is neither loaded nor stored
  const int cols = (!W_MN && p.tile_n > 0) ? p.tile_n : 32 * NW;
  const int n0 = blockIdx.x * cols;
  const int bz = blockIdx.y;

  const typename T::storage* X = (const typename T::storage*)p.A + (long long)bz * p.sab;
  const typename T::storage* W = (const typename T::storage*)p.B + (long long)bz * p.sbb;

  // both operands through bounds-checked buffers: rows >= N (>= M) and k >= K read zero
  const uint32_t w_bytes = W_MN ? (uint32_t)(((long long)(p.K - 1) * p.sbk + p.N) * ES)
                                : (uint32_t)(((long long)(p.N - 1) * p.sbn + p.K) * ES);
  const uint64_t wp = reinterpret_cast<uint64_t>(W);
  const u32x4_t rw = {(uint32_t)wp, (uint32_t)(wp >> 32) & 0xffffu, w_bytes, 0x00020000u};
  const uint32_t x_bytes = (uint32_t)(((long long)(p.M - 1) * p.sam + p.K) * ES);
  const uint64_t xp = reinterpret_cast<uint64_t>(X);
  const u32x4_t rx = {(uint32_t)xp, (uint32_t)(xp >> 32) & 0xffffu, x_bytes, 0x00020000u};

  // A load instruction covers 8 rows x 128 contiguous bytes (8 lanes per row); the lane fetches
  // the 16-byte chunk that belongs at its landing position (chunk c of row r sits at
  // c ^ ((r >> 1) & 7)).  (row >> 1) & 7 only depends on the lane, not on which group of 8 rows.
  const int lrow = lane >> 3;
  const int lchunk = (lane & 7) ^ ((lrow >> 1) & 3) ^ 0;   // rows 8 i + lrow: ((8 i + lrow) >> 1) & 7 = 4 (i & 1) + (lrow >> 1)
  uint32_t wvoff[4 * NW], xvoff[XR / 8];
  int wchunk[4 * NW], xchunk[XR / 8];
#pragma unroll
  for (int i = 0; i < 4 * NW; ++i) {
    const int row = 8 * i + lrow;
    if (W_MN) {
      // load i covers 1024 / RB k rows of the block; the lane fetches the chunk of 8 columns that
      // belongs at its landing position.  wchunk holds the k row (for the tail test).
      const int krow = (1024 / RB) * i + lane / (RB / 16);
      const int pos = lane % (RB / 16);
      const int c = NW == 2 ? pos ^ (((krow >> 1) & 1) << 2) : pos;
      const int n = n0 + EPC * c;
      wchunk[i] = krow;
      wvoff[i] = n < p.N ? (uint32_t)(((long long)krow * p.sbk + n) * ES) : SK_OOB;
    } else {
      wchunk[i] = (lane & 7) ^ ((row >> 1) & 7);
      const int n = n0 + row;
      wvoff[i] = (n < p.N && row < cols) ? (uint32_t)(((long long)n * p.sbn + wchunk[i] * EPC) * ES) : SK_OOB;
    }
  }
#pragma unroll
  for (int i = 0; i < XR / 8; ++i) {
    const int row = 8 * i + lrow;
    xchunk[i] = (lane & 7) ^ ((row >> 1) & 7);
    xvoff[i] = row < p.M ? (uint32_t)(((long long)row * p.sam + xchunk[i] * EPC) * ES) : SK_OOB;
  }
  (void)lchunk;
  const uint32_t my_ring = lds + (uint32_t)wave * (DEPTH * Shape::SLOT);

  // fragment read address inside a region: row r, chunk 2 s + h, swizzled
  uint32_t rd[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) rd[s] = (uint32_t)(r * 128 + (((2 * s + h) ^ ((r >> 1) & 7)) << 4));
  const bool x_lane = XR >= 32 || r < XR;   // lanes of rows that are not staged hold zero operands
  // n-contiguous weight: the lane's address for the transposing read of column tile t at k slice 0
  // (k row 8 h + e, columns 32 t + 16 (g & 1) + 4 q .. + 3); k slice s is 16 k rows further, the
  // second half of the lane's eight k values four k rows.  With 64-byte rows the four k rows a half
  // wave reads are 256 contiguous bytes and need no swizzle.
  uint32_t rdw[2];
  {
    const int g = lane >> 4, e = (lane >> 2) & 3, q = lane & 3;
    const int krow = 8 * (g >> 1) + e;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int mn = 32 * t + 16 * (g & 1) + 4 * q;
      const int chunk = NW == 2 ? (mn >> 3) ^ (((krow >> 1) & 1) << 2) : (mn >> 3);
      rdw[t] = (uint32_t)(krow * RB + chunk * 16 + ((mn >> 2) & 1) * 8);
    }
  }

  const int KB = (p.K + KBE - 1) / KBE;   // k blocks in total; this wave takes wave, wave + 4, ...
  const int k_chunks = p.K / EPC;          // valid 16-byte chunks per row

  auto issue = [&](int kb, int slot) {
    const bool live = kb < KB;
    const uint32_t base = my_ring + (uint32_t)slot * Shape::SLOT;
    const uint32_t soff = (uint32_t)kb * 128u;   // bytes of a block per row
    const uint32_t soff_w = W_MN ? (uint32_t)kb * (uint32_t)(KBE * ES) * (uint32_t)p.sbk : soff;
#pragma unroll
    for (int i = 0; i < 4 * NW; ++i) {
      const bool in_k = live && (W_MN ? kb * KBE + wchunk[i] < p.K : (kb * 8 + wchunk[i]) < k_chunks);
      sk_load_to_lds<true>(rw, base + (uint32_t)i * 1024u, in_k ? wvoff[i] : SK_OOB, soff_w);
    }
#pragma unroll
    for (int i = 0; i < XR / 8; ++i) {
      const bool in_k = live && (kb * 8 + xchunk[i]) < k_chunks;
      sk_load_to_lds<false>(rx, base + SK_WBYTES + (uint32_t)i * 1024u, in_k ? xvoff[i] : SK_OOB, soff);
    }
  };

  f32x16_t acc[NW][MT];
#pragma unroll
  for (int t = 0; t < NW; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[t][mt][v] = 0.0f;

  // This wave's k blocks are wave, wave + 4, ... (count of them); it walks them in rotated
  // order, starting at a block that depends on the workgroup, so that the workgroups resident at
  // one time are spread over different byte offsets of their rows -- with rows a power of two
  // apart, all workgroups reading the same offset would hammer the same few memory channels.
  const int count = KB > wave ? (KB - wave + SK_WAVES - 1) / SK_WAVES : 0;
  // (An n-contiguous weight is walked in step instead: neighbouring workgroups then read neighbouring
  // 128-byte pieces of the same k rows at about the same time.)
  const int rot = (!W_MN && count > 0) ? (int)((blockIdx.x * 7u) % (unsigned)count) : 0;
  auto block_at = [&](int j) {   // j-th block of the walk, or KB (= nothing) past the end
    if (j >= count) return KB;
    int jj = j + rot;
    if (jj >= count) jj -= count;
    return wave + SK_WAVES * jj;
  };

#pragma unroll
  for (int d = 0; d < DEPTH; ++d) issue(block_at(d), d);

  // Each trip consumes DEPTH blocks; block d of the trip was issued DEPTH blocks ago.  Loads
  // retire in order and every block issues exactly LOADS of them (out-of-range ones included),
  // so a block has landed once at most LOADS (DEPTH - 1) younger loads remain outstanding.
  for (int j0 = 0; j0 < count; j0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int j = j0 + d;
      asm volatile("s_waitcnt vmcnt(%0)" : : "i"(Shape::LOADS * (DEPTH - 1)) : "memory");
      const uint32_t base = my_ring + (uint32_t)d * Shape::SLOT;
      u32x4_t wf[NW][4], xf[MT][4];
#pragma unroll
      for (int s = 0; s < 4; ++s) {
#pragma unroll
        for (int t = 0; t < NW; ++t) {
          if constexpr (W_MN && ES == 4) {
            // fp32: the four k rows 8 s + 4 h + 0..3 of column r, one dword each (the half waves meet on the same
            // banks, 512 bytes apart: two passes per read, of sixteen reads per block against sixteen MFMAs)
            const uint32_t a = base + (uint32_t)((8 * s + 4 * h) * RB + r * 4);
            wf[t][s] = u32x4_t{*reinterpret_cast<const SRT_LDS uint32_t*>(a), *reinterpret_cast<const SRT_LDS uint32_t*>(a + RB),
                               *reinterpret_cast<const SRT_LDS uint32_t*>(a + 2 * RB),
                               *reinterpret_cast<const SRT_LDS uint32_t*>(a + 3 * RB)};
          } else if constexpr (W_MN) {
            const uint32_t a = base + rdw[t & 1] + s * (16 * RB);
            const u32x2_t lo = __builtin_bit_cast(
                u32x2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<SRT_LDS s16x4_t*>(a)));
            const u32x2_t hi = __builtin_bit_cast(
                u32x2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<SRT_LDS s16x4_t*>(a + 4 * RB)));
            wf[t][s] = u32x4_t{lo.x, lo.y, hi.x, hi.y};
          } else {
            wf[t][s] = *reinterpret_cast<const SRT_LDS u32x4_t*>(base + t * SK_WTILE + rd[s]);
          }
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          u32x4_t x = {0u, 0u, 0u, 0u};
          if (x_lane) x = *reinterpret_cast<const SRT_LDS u32x4_t*>(base + SK_WBYTES + mt * 4096 + rd[s]);
          xf[mt][s] = x;
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // fragments are in registers: the slot is free
      issue(block_at(j + DEPTH), d);
      if (j < count) {
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
          for (int t = 0; t < NW; ++t)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[t][mt] = mfma32s<T>(xf[mt][s], wf[t][s], acc[t][mt]);
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();   // every wave's loads have landed and its ring is idle: reuse LDS for the reduction

  float* red = reinterpret_cast<float*>(sk_lds_raw);   // [NW x MT tiles][4 waves][16][64] = NW x MT x 16 KiB
#pragma unroll
  for (int t = 0; t < NW; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int v = 0; v < 16; ++v) red[(((t * MT + mt) * SK_WAVES + wave) * 16 + v) * 64 + lane] = acc[t][mt][v];
  __syncthreads();

  // wave w finishes accumulator registers 4w .. 4w+3: rows m = 8 w + 4 h + i, column n
  Epilogue<T> ep(p);
  typename T::storage* C = (typename T::storage*)p.C + (long long)bz * p.scb;
#pragma unroll
  for (int t = 0; t < NW; ++t) {
    const int n = n0 + 32 * t + r;
    if (n >= p.N || 32 * t + r >= cols) continue;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int mb = 32 * mt + 8 * wave + 4 * h;
      float out[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int v = 4 * wave + i;
        float s = 0.0f;
#pragma unroll
        for (int w = 0; w < SK_WAVES; ++w) s += red[(((t * MT + mt) * SK_WAVES + w) * 16 + v) * 64 + lane];
        out[i] = s;
      }
      ep.finish_run(out, [&](int i, int* m, int* nn) {
        *m = mb + i;
        *nn = n;
        return *m < p.M;
      });
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (mb + i < p.M) C[(long long)(mb + i) * p.scm + (long long)n * p.scn] = T::from_float(out[i]);
    }
  }
}

template <typename T, int XR, int NW, bool W_MN = false>
hipError_t launch_skinny_shape(const GemmProblem& p, hipStream_t stream) {
  auto kernel = gemm_skinny_kernel<T, XR, NW, W_MN>;
  constexpr int lds_bytes = SkinnyShape<XR, NW>::LDS;
  static std::atomic<uint32_t> configured{0};
  if (hipError_t e = ensure_lds_limit(reinterpret_cast<const void*>(kernel), lds_bytes, configured); e != hipSuccess) return e;
  const int cols = (!W_MN && p.tile_n > 0) ? p.tile_n : 32 * NW;
  hipLaunchKernelGGL(kernel, dim3((p.N + cols - 1) / cols, p.batch), dim3(SK_WAVES * 64), lds_bytes, stream, p);
  return launch_status(stream);
}

template <typename T>
hipError_t launch_skinny_type16(const GemmProblem& p, hipStream_t stream);

template <typename T>
hipError_t launch_skinny_type(const GemmProblem& p, hipStream_t stream) {
  if constexpr (sizeof(typename T::storage) == 4) {
    // fp32: the k-contiguous weight, up to 32 rows.  A block of 128 bytes per row is 32 k and sixteen MFMAs per tile,
    // eight times the matrix time per byte of a 16-bit type: two tiles per workgroup would leave it bound by the matrix
    // pipe with one workgroup per unit, so the form is always one tile, two workgroups per unit.
    if (p.sbk != 1) {   // n-contiguous weight: 32 columns per workgroup are whole 128-byte lines of a k row
      if (p.M <= 8) return launch_skinny_shape<T, 8, 1, true>(p, stream);
      if (p.M <= 16) return launch_skinny_shape<T, 16, 1, true>(p, stream);
      return launch_skinny_shape<T, 32, 1, true>(p, stream);
    }
    if (p.M <= 8) return launch_skinny_shape<T, 8, 1>(p, stream);
    if (p.M <= 16) return launch_skinny_shape<T, 16, 1>(p, stream);
    return launch_skinny_shape<T, 32, 1>(p, stream);
  } else {
    return launch_skinny_type16<T>(p, stream);
  }
}

template <typename T>
hipError_t launch_skinny_type16(const GemmProblem& p, hipStream_t stream) {
  if (p.sbk != 1) {   // n-contiguous weight
    // Always 64 columns per workgroup, i.e. whole 128-byte lines of a k row.  (With 32 columns the
    // two workgroups that share a line each pull it from memory: 11008 columns x 4096 took 39 us
    // instead of 22 us, 8192 x 8192 47 us instead of 40 us.)
    if (p.M <= 8) return launch_skinny_shape<T, 8, 2, true>(p, stream);
    if (p.M <= 16) return launch_skinny_shape<T, 16, 2, true>(p, stream);
    if (p.M <= 32) return launch_skinny_shape<T, 32, 2, true>(p, stream);
    return launch_skinny_shape<T, 64, 2, true>(p, stream);
  }
  if (p.M <= 8) return launch_skinny_shape<T, 8, 1>(p, stream);
  if (p.M <= 16) return launch_skinny_shape<T, 16, 1>(p, stream);
  // two W tiles per workgroup once that still gives most CUs a workgroup (192 of them)
  const long long wide_groups = (long long)((p.N + 63) / 64) * p.batch;
  // One such workgroup fits a compute unit, so with fewer workgroups than units the rest idle and the weight
  // streams that much slower (14336 columns: 224 workgroups of 64, 23.5 us; the kernel of 32 columns, two
  // workgroups per unit, is no better because x then crosses L2 -> LDS twice as often).  When the columns
  // allow, the tile is narrowed to a multiple of 8 columns that gives every unit one workgroup: 14336 = 256 x 56.
  GemmProblem q = p;
  if (wide_groups >= 192 && p.batch == 1) {
    const int cus = compute_units();
    const int even = 8 * (int)((p.N + 8LL * cus - 1) / (8LL * cus));
    if (even > 32 && even < 64) q.tile_n = even;
  }
  if (p.M <= 32) {
    if (wide_groups >= 192) return launch_skinny_shape<T, 32, 2>(q, stream);
    return launch_skinny_shape<T, 32, 1>(p, stream);
  }
  if (wide_groups >= 192) return launch_skinny_shape<T, 64, 2>(q, stream);
  return launch_skinny_shape<T, 64, 1>(p, stream);
}

inline bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

}  // namespace

bool skinny_supported(const GemmProblem& p) {
  if (p.dtype == srtReal32F) {
    // fp32: up to 32 rows against a k-contiguous weight; the same conditions at four elements per 16-byte chunk
    if (p.M > 32 || p.M < 1 || p.K < 1 || p.N < 32 || p.batch > 65535) return false;
    if (p.sak != 1 || (p.K % 4) != 0) return false;
    if ((p.sam % 4) != 0 && p.M > 1) return false;
    if ((p.sab % 4) != 0 || (p.sbb % 4) != 0) return false;
    if (p.sam < 0 || p.scm < 0 || p.scn < 0) return false;
    if (!aligned16(p.A) || !aligned16(p.B)) return false;
    if (((long long)p.M + 8) * p.sam + p.K >= (0x7fffffffLL / 4 - 4096)) return false;
    if (p.sbk == 1 && p.sbn != 1) {                     // W k-contiguous ([N, K])
      if ((p.sbn % 4) != 0 || p.sbn < 0) return false;
      return ((long long)p.N + 32) * p.sbn + p.K < (0x7fffffffLL / 4 - 4096);
    }
    if (p.sbn != 1 || (p.N % 4) != 0) return false;     // W n-contiguous ([K, N]): whole 16-byte chunks of a k row
    if (p.sbk < 4 || (p.sbk % 4) != 0) return false;
    return ((long long)p.K + 32) * p.sbk + p.N < (0x7fffffffLL / 4 - 4096);
  }
  if (p.dtype != srtReal16BF && p.dtype != srtReal16F) return false;
  if (p.M > 64 || p.M < 1 || p.K < 1) return false;
  if (p.sak != 1) return false;                         // x is k-contiguous
  if ((p.K % 8) != 0) return false;                     // whole 16-byte chunks
  if ((p.sam % 8) != 0 && p.M > 1) return false;
  if ((p.sab % 8) != 0 || (p.sbb % 8) != 0) return false;
  if (p.sam < 0 || p.scm < 0 || p.scn < 0) return false;
  if (!aligned16(p.A) || !aligned16(p.B)) return false;
  if (p.batch > 65535) return false;
  // 32-bit byte offsets must reach every row of x too (a row view of a wide tensor has a large pitch)
  if (((long long)p.M + 8) * p.sam + p.K >= (0x7fffffffLL / 2 - 4096)) return false;
  if (p.sbk == 1) {                                     // W k-contiguous ([N, K])
    if ((p.sbn % 8) != 0 && p.N > 1) return false;
    if (p.sbn < 0) return false;
    // 32-bit byte offsets must reach every row of W (and stay below the out-of-range marker)
    if (((long long)p.N + 32) * p.sbn + p.K >= (0x7fffffffLL / 2 - 4096)) return false;
  } else {                                              // W n-contiguous ([K, N])
    if (p.sbn != 1 || (p.N % 8) != 0) return false;     // whole 16-byte chunks of a k row
    if (p.sbk < 8 || (p.sbk % 8) != 0) return false;
    if (((long long)p.K + 64) * p.sbk + p.N >= (0x7fffffffLL / 2 - 4096)) return false;
  }
  // worth it only when the weight dominates the traffic
  return p.N >= 32;
}

// Whether the heuristic takes this kernel for a problem it supports.  Up to M = 32 always.  With
// 33..64 rows a workgroup needs 128-144 KiB of LDS, one fits per compute unit, and the kernel pays
// only when its workgroups run in a single round that keeps most units streaming: 192..256
// workgroups of 64 weight rows (64 x 14336 x 4096: 26.5 us against 32 us for split-K), or at most
// 256 of 32 rows unless they are few and the k loop is long (64 x 4096 x 4096, 128 workgroups: 17 us
// against 21 us; 64 x 4096 x 14336: 51 us against 35 us; 64 x 11008 x 4096, 344 workgroups: 34 us
// against 29 us; 64 x 32768 x 1024: 22 us against 17 us for 64 x 64 tiles).
//
// An n-contiguous weight streams at 4.3-4.8 TB/s at best (x . W with 14336 x 4096: 25-28 us for up
// to 32 rows, where split-K takes 29 us and the k-contiguous form of this kernel 21 us), always with
// 64 columns per workgroup, so it needs its workgroups to number at most one round, and a short k
// loop when they are few; deeper problems go to split-K (8 x 4096 x 8192: 25 us against 37 us; 8 x 1024 x 8192: 21 against 36)
// and more than 256 workgroups to the 128 x 256 tiles (8 x 28672 x 1024: 16 us against 19 us).
bool skinny_preferred(const GemmProblem& p) {
  // fp32 (up to 32 rows): ahead of every other fp32 kernel on 80 shapes x . W^T of 1-32 rows, 256-32768 columns and
  // K 256-8192 -- 1 x 14336 x 4096 43 us = 5.5 TB/s against 71 on 64 x 64 tiles and 86 on the 32 x 32 kernel, 8 x 4096 x 4096
  // 24.5 against 67, 32 x 32768 x 256 11.7 against 12.2 -- and on 48 shapes x . W, where the 32 x 32 kernel has 16-byte loads
  // (1 x 14336 x 4096 47 us against 57, 8 x 4096 x 4096 25.8 against 36.6, 32 x 14336 x 4096 a tie at 59.5) -- so always, short of
  // the many short k loops of a large batch, where the 16-bit form loses (below) and the fp32 one has not been measured
  if (p.dtype == srtReal32F) return !((long long)((p.N + 31) / 32) * p.batch > (p.batch > 1 ? 512 : 1024) && p.K < 2048);
  // more than 32 rows, a k loop of a few blocks and many workgroups: the two-tile form's set-up does
  // not pay (64 x 14336 x 64: 7.3 us against 5.5 us for 64 x 64 tiles; K = 256: 7.9 against 6.8; but
  // 64 x 3072 x 256: 5.9 against 6.6)
  if (p.M > 32 && p.K < 512 && (long long)((p.N + 31) / 32) * p.batch > 128) return false;
  // many rounds of workgroups with a short k loop each (a large batch): the per-workgroup set-up and
  // reduction dominate (32 x 32 x 4096 x 512: 52 us against 28 us for 128 x 256 tiles)
  // (from 512 workgroups in a batch: 36 x 8 x 768 x 328 10.6 us against 8.3 for 64 x 64 tiles, 12 x 28 x 2256 x 1512 27 against 21)
  if ((long long)((p.N + 31) / 32) * p.batch > (p.batch > 1 ? 512 : 1024) && p.K < 2048) return false;
  if (p.sbk != 1) {
    const long long groups = (long long)((p.N + 63) / 64) * p.batch;
    if (groups > 256) return false;
    if (p.K <= 2048) return true;
    if (p.K <= 4096) return p.M <= 16 || groups <= 32 || groups >= (p.M <= 32 ? 192 : 224);
    return false;
  }
  if (p.M <= 32) return true;
  const long long groups64 = (long long)((p.N + 63) / 64) * p.batch, groups32 = (long long)((p.N + 31) / 32) * p.batch;
  if (groups64 >= 192) return groups64 <= 256;
  if (groups32 > 256) return false;
  return groups32 >= 192 || p.K <= 4096;
}

hipError_t launch_skinny(const GemmProblem& p, hipStream_t stream) {
  if (p.dtype == srtReal32F) return launch_skinny_type<F32>(p, stream);
  if (p.dtype == srtReal16BF) return launch_skinny_type<BF16>(p, stream);
  return launch_skinny_type<F16>(p, stream);
}

}  // namespace srt
