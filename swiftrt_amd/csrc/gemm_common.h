// Shared definitions for the matmul kernels: the normalized problem, element codecs and
// the fused bias + activation epilogue.  gfx950 only.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <chrono>
#include <random>

#include "../../include/srt_hip.h"
#include "status.h"

namespace srt {

// A matmul after the caller's transposes, orders and views have been folded into strides.
// op(A)[m,k] = A[m*sam + k*sak], op(B)[k,n] = B[k*sbk + n*sbn], C[m,n] = C[m*scm + n*scn];
// batch b adds b*sab / b*sbb / b*scb.  All strides are in elements.
struct GemmProblem {
  int dtype;  // srtDataType
  int M, N, K, batch;
  const void* A;
  const void* B;
  void* C;
  const void* bias;  // may be null
  long long sam, sak, sab;
  long long sbk, sbn, sbb;
  long long scm, scn, scb;
  long long sbias;  // stride between bias elements
  int bias_per_row;  // 0: bias indexed by column n (the Dense case); 1: by row m (after a C^T flip)
  int activation;    // srtActivation
  float coef;
  int tile_n;        // kernel-specific: columns per workgroup when a launcher narrows its tile (0: the kernel's own)
};

// ---- element codecs ---------------------------------------------------------------------
struct BF16 {
  using storage = uint16_t;
  static constexpr int dtype = srtReal16BF;
  static __device__ __forceinline__ float to_float(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
  // round to nearest even; NaN -> 0x7FFF.  Same rule as BFloat16.float2bfloat16_rn in the
  // reference (platform/common/BFloat16.swift:53-80).
  static __device__ __forceinline__ uint16_t from_float(float f) {
    uint32_t x = __float_as_uint(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return 0x7fff;
    return (uint16_t)((x + 0x7fffu + ((x >> 16) & 1u)) >> 16);
  }
  // Two values -> one dword (a in the low half).  EXACT = false uses the hardware converter
  // (round to nearest even, one instruction) and is only valid when neither input is a NaN;
  // EXACT = true is the scalar encoder (NaN -> 0x7FFF).  Callers test a whole tile for NaNs once
  // and pick the variant.
  template <bool EXACT>
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    if (EXACT) return (uint32_t)from_float(a) | ((uint32_t)from_float(b) << 16);
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    f32x2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
  }
};

// V fp32 values (V even) -> V bfloat16 in V / 2 dwords, bit for bit what BF16::from_float gives for each: when none
// of them is a NaN (one unordered compare per pair) the hardware converter does two values per instruction;
// the scalar encoder (NaN -> 0x7FFF) runs only for a lane that holds a NaN.
template <int V>
__device__ __forceinline__ void encode_bf16(const float (&r)[V], uint32_t (&w)[V / 2]) {
  static_assert(V % 2 == 0, "pairs");
  bool clean = true;
#pragma unroll
  for (int i = 0; i < V; i += 2) clean &= !__builtin_isunordered(r[i], r[i + 1]);
  if (clean) {
#pragma unroll
    for (int i = 0; i < V; i += 2) w[i / 2] = BF16::pack2<false>(r[i], r[i + 1]);
  } else {
#pragma unroll
    for (int i = 0; i < V; i += 2) w[i / 2] = BF16::pack2<true>(r[i], r[i + 1]);
  }
}

struct F16 {
  using storage = uint16_t;
  static constexpr int dtype = srtReal16F;
  static __device__ __forceinline__ float to_float(uint16_t h) {
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;
  }
  static __device__ __forceinline__ uint16_t from_float(float f) {
    _Float16 v = (_Float16)f;  // v_cvt_f16_f32: round to nearest even
    uint16_t h;
    __builtin_memcpy(&h, &v, 2);
    return h;
  }
  template <bool EXACT>
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    return (uint32_t)from_float(a) | ((uint32_t)from_float(b) << 16);
  }
};

struct F32 {
  using storage = float;
  static constexpr int dtype = srtReal32F;
  static __device__ __forceinline__ float to_float(float v) { return v; }
  static __device__ __forceinline__ float from_float(float v) { return v; }
};

// ---- epilogue ---------------------------------------------------------------------------
// Activation on the fp32 accumulator.  Definitions follow the reference where it has one
// (sigmoid: CpuMath.swift:1369-1377; tanh: libm) and cuDNN's for the rest.
__device__ __forceinline__ float apply_activation(int activation, float coef, float x) {
  switch (activation) {
    case srtActivationSigmoid: return 1.0f / (1.0f + expf(-x));
    case srtActivationRelu: return x > 0.0f ? x : 0.0f;
    case srtActivationTanh: return tanhf(x);
    case srtActivationClippedRelu: {
      float y = x > 0.0f ? x : 0.0f;
      return y < coef ? y : coef;
    }
    case srtActivationElu: return x > 0.0f ? x : coef * (expf(x) - 1.0f);
    default: return x;
  }
}

// The same for results stored in a 16-bit type: the hardware exponential and reciprocal (a few
// fp32 ulps: 2^-13 of a half's rounding step, 2^-16 of a bfloat16's) instead of libm's expf / tanhf,
// whose range reduction and branches cost ten times the instructions -- fused into a 256 x 256
// tile's epilogue, libm's tanh took longer than the whole k loop at K = 4096.  Where a closed
// form cancels (exp(x) - 1 near 0) a short series takes over, so the relative error stays
// at fp32 rounding level everywhere.  NaN in, NaN out; +-inf give the limits.
// tanh has no exponential at all: the epilogues are bound by the vector unit, where an exponential or a
// reciprocal costs four ordinary instructions, and 1 - 2 / (exp(2|x|) + 1) with its series near 0 came to 88
// issue cycles per element (14 us of a 256 x 256 tile's epilogue).  Instead x P(x^2) / Q(x^2) with P and Q of
// degree 2, fitted to tanh on [0, 4.97] (largest relative error 5.5e-5: an eighth of a half's rounding step, a
// seventieth of a bfloat16's), and +-1 beyond -- where tanh is within 1e-4 of 1, and rounds to 1 in both types as
// the quotient's value at 4.97 does: 56 cycles.  Exact at 0 (x P(0) / Q(0) = x), relative error uniform down to
// the smallest arguments.
template <int ACT>
__device__ __forceinline__ float activation16_ct(float coef, float x) {
  // fused multiply-adds here whatever the translation unit's setting (the element-wise kernels are compiled
  // without contraction for their basic operations): three instructions fewer per tanh, and the same bits
  // as the GEMM epilogues' use of this function
#pragma clang fp contract(fast)
  if (ACT == srtActivationSigmoid) return __fdividef(1.0f, 1.0f + __expf(-x));
  if (ACT == srtActivationTanh) {
    const float x2 = x * x;
    const float num = x * ((0.00068074085f * x2 + 0.102823904f) * x2 + 1.0f);
    const float den = (0.012931462f * x2 + 0.43594227f) * x2 + 1.0f;
    const float r = num * __builtin_amdgcn_rcpf(den);
    // (a NaN fails the comparison and comes out of the quotient as a NaN; for huge |x| the quotient is not used)
    return fabsf(x) > 4.97f ? copysignf(1.0f, x) : r;
  }
  if (ACT == srtActivationElu) {
    const float x2 = x * x;
    const float series = x + x2 * (0.5f + x * (0.16666667f + x * (0.041666668f + x * 0.008333334f)));
    const float em1 = x > -0.125f ? series : __expf(x) - 1.0f;
    return x > 0.0f ? x : coef * em1;
  }
  return x;
}
__device__ __forceinline__ float apply_activation_16(int activation, float coef, float x) {
  switch (activation) {
    case srtActivationSigmoid: return activation16_ct<srtActivationSigmoid>(coef, x);
    case srtActivationTanh: return activation16_ct<srtActivationTanh>(coef, x);
    case srtActivationElu: return activation16_ct<srtActivationElu>(coef, x);
    default: return apply_activation(activation, coef, x);
  }
}

// Same with the activation fixed at compile time: kernels switch on the activation once per
// workgroup and run an epilogue specialised for it, so the unrolled store code of the common
// cases (identity, relu) carries no transcendental code and no per-element branches.
template <int ACT>
__device__ __forceinline__ float activation_ct(float coef, float x) {
  if (ACT == srtActivationSigmoid) return 1.0f / (1.0f + expf(-x));
  if (ACT == srtActivationRelu) return x > 0.0f ? x : 0.0f;
  if (ACT == srtActivationTanh) return tanhf(x);
  if (ACT == srtActivationClippedRelu) {
    float y = x > 0.0f ? x : 0.0f;
    return y < coef ? y : coef;
  }
  if (ACT == srtActivationElu) return x > 0.0f ? x : coef * (expf(x) - 1.0f);
  return x;
}

// Epilogue state for one output column (or row) set; bias is read as element type T.
template <typename T>
struct Epilogue {
  const typename T::storage* bias;
  long long sbias;
  int per_row;
  int activation;
  float coef;
  __device__ __forceinline__ explicit Epilogue(const GemmProblem& p)
      : bias((const typename T::storage*)p.bias), sbias(p.sbias), per_row(p.bias_per_row),
        activation(p.activation), coef(p.coef) {}
  __device__ __forceinline__ float bias_at(int m, int n) const {
    if (!bias) return 0.0f;
    return T::to_float(bias[(long long)(per_row ? m : n) * sbias]);
  }
  __device__ __forceinline__ typename T::storage finish(float acc, float b) const {
    float v = acc + b;
    if (activation != srtActivationIdentity)
      v = sizeof(typename T::storage) == 2 ? apply_activation_16(activation, coef, v) : apply_activation(activation, coef, v);
    return T::from_float(v);
  }

  // The same for a run of COUNT sums of one lane, in place and still in fp32 (the caller rounds and stores):
  // v[q] = activation(v[q] + bias), where at(q, &m, &n) gives the element's place and whether it exists.  The bias
  // values are fetched first and the run ends before the caller's first store: loads and stores share one counter,
  // so a store that follows a (conditional) load of its own waits for every earlier store's acknowledgement, and a
  // lane's stores then go out one round trip apart.  Identity and relu are switched once per run, not per element.
  template <int ACT, bool BIAS, int COUNT, typename At>
  __device__ __forceinline__ void finish_run_ct(float (&v)[COUNT], At&& at) const {
    float b[COUNT];
#pragma unroll
    for (int q = 0; q < COUNT; ++q) {
      b[q] = 0.0f;
      if constexpr (BIAS) {
        int m = 0, n = 0;
        if (at(q, &m, &n)) b[q] = T::to_float(bias[(long long)(per_row ? m : n) * sbias]);
      }
    }
#pragma unroll
    for (int q = 0; q < COUNT; ++q) v[q] = activation_ct<ACT>(coef, v[q] + b[q]);
  }
  template <int COUNT, typename At>
  __device__ __forceinline__ void finish_run(float (&v)[COUNT], At&& at) const {
    if (activation == srtActivationIdentity) {
      if (bias) finish_run_ct<srtActivationIdentity, true>(v, at);
      else finish_run_ct<srtActivationIdentity, false>(v, at);
    } else if (activation == srtActivationRelu) {
      if (bias) finish_run_ct<srtActivationRelu, true>(v, at);
      else finish_run_ct<srtActivationRelu, false>(v, at);
    } else {
      float b[COUNT];
#pragma unroll
      for (int q = 0; q < COUNT; ++q) b[q] = 0.0f;
      if (bias) {
#pragma unroll
        for (int q = 0; q < COUNT; ++q) {
          int m = 0, n = 0;
          if (at(q, &m, &n)) b[q] = T::to_float(bias[(long long)(per_row ? m : n) * sbias]);
        }
      }
#pragma unroll
      for (int q = 0; q < COUNT; ++q)
        v[q] = sizeof(typename T::storage) == 2 ? apply_activation_16(activation, coef, v[q] + b[q])
                                                : apply_activation(activation, coef, v[q] + b[q]);
    }
  }
};

// Raises a kernel's dynamic-LDS limit above the 64 KiB default, once per device (the attribute
// belongs to the kernel's image on the current device).  `done` holds one bit per device.
inline hipError_t ensure_lds_limit(const void* kernel, int bytes, std::atomic<uint32_t>& done) {
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  const uint32_t bit = 1u << (device & 31);
  if (done.load(std::memory_order_relaxed) & bit) return hipSuccess;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess) done.fetch_or(bit, std::memory_order_relaxed);
  return e;
}

// Compute units of the current device (cached per device).
inline int compute_units() {
  static std::atomic<int> cached[32];
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return 256;
  int n = cached[device & 31].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || n <= 0) n = 256;
    cached[device & 31].store(n, std::memory_order_relaxed);
  }
  return n;
}

// Flag values of kernels whose workgroups tell each other "my part is in memory" (the tail-sharing matmul): a 64-bit
// launch counter that starts at a value drawn once per process.  The flags live in
// memory that other kernels have written before (the allocator recycles blocks), so what they hold at launch
// is arbitrary -- most likely the flags of an earlier launch of this kernel.  Those hold earlier values of the
// counter, which this launch's value differs from by construction (2^64 launches apart at the earliest);
// anything else -- other kernels' data, another process's flags in memory the driver handed over -- matches
// with probability 2^-64 per flag.
inline unsigned long long next_launch_epoch() {
  static const unsigned long long start = [] {
    std::random_device rd;
    unsigned long long v = ((unsigned long long)rd() << 32) ^ (unsigned long long)rd();
    v ^= (unsigned long long)std::chrono::steady_clock::now().time_since_epoch().count() * 0x9e3779b97f4a7c15ull;
    return v;
  }();
  static std::atomic<unsigned long long> counter{0};
  return start + ++counter;
}

// ---- launchers (one per kernel family), defined in the .hip files ------------------------
// Each returns hipSuccess/hip error from the launch; `name` receives the kernel family.
bool generic_supported(const GemmProblem& p);
hipError_t launch_generic(const GemmProblem& p, hipStream_t stream);

// Tile configuration chosen for the MFMA family, or 0 if the problem does not qualify.
int mfma_select(const GemmProblem& p);
// Same for a caller-chosen tile (1: 256 x 256, 2: 128 x 128, 3: 64 x 64, 4: 256 x 256 with 64-deep
// stages, 5: 256 x 256 on 16x16x32 MFMAs); 0 if it does not qualify.
int mfma_config(const GemmProblem& p, int tile);
const char* mfma_name(int config);
hipError_t launch_mfma(const GemmProblem& p, int config, hipStream_t stream);
// Split-K over the 256 x 256 kernel: number of k parts (0: the problem does not qualify) and launch.
int mfma_splitk_parts(const GemmProblem& p);
bool mfma_prefers_splitk(const GemmProblem& p);
bool mfma_prefers_tail(const GemmProblem& p);
bool mfma_prefers_quarter(const GemmProblem& p);
hipError_t launch_mfma_splitk(const GemmProblem& p, hipStream_t stream);

bool skinny_supported(const GemmProblem& p);
bool skinny_preferred(const GemmProblem& p);   // the heuristic's choice among the problems it supports
hipError_t launch_skinny(const GemmProblem& p, hipStream_t stream);

bool f32_mfma_supported(const GemmProblem& p);
hipError_t launch_f32_mfma(const GemmProblem& p, hipStream_t stream);
bool f32_mfma_prefers_splitk(const GemmProblem& p);
hipError_t launch_f32_mfma_variant(const GemmProblem& p, bool splitk, hipStream_t stream);
bool f32_ring_fits(const GemmProblem& p);
int f32_ring_choice(const GemmProblem& p);   // among the fp32 kernels, for a problem f32_ring_fits admits
hipError_t launch_f32_ring(const GemmProblem& p, hipStream_t stream, int shape);
int f32_tile_parts(const GemmProblem& p);
hipError_t launch_f32_tile_parts(const GemmProblem& p, hipStream_t stream);

}  // namespace srt
