// Element-wise neighbours of the matmul path on the device: add / sub / mul / div / max / min
// (tensor-tensor and tensor-element), neg, exp, sigmoid, tanh, copy with type conversion, fill.
// They let the recurrent cells (tanh(matmul + bias), the LSTM gate arithmetic) and the unfused
// Dense neighbours run without a host round trip.
//
// All of them are bandwidth-bound maps, so there is ONE kernel: operands are described by a
// collapsed strided index space (broadcast = stride 0), a lane moves V consecutive elements of the
// innermost dimension as one 16-byte (or 8-byte) access when layout and alignment allow (V = 1
// otherwise), arithmetic is fp32 and the result is rounded once to the element type -- the
// reference's CPU definitions evaluated in E.Value (Sources/SwiftRTCore/platform/cpu/functions/
// CpuMath.swift: add :646-662, mul :1235-1256, max :1189-1209 `a >= b ? a : b`, sigmoid
// :1369-1377 `1 / (1 + exp(-x))`, ...).  This file is compiled with floating-point contraction
// off so the four basic operations match a C restatement bit for bit.
#include <cstring>

#include "gemm_common.h"
#include "status.h"

namespace srt {
namespace ew {

constexpr int MAX_RANK = 4;   // after collapsing adjacent dimensions
constexpr int kVectorsPerLane = 4;   // (two: sigmoid 32.2 -> 30.7 us, bias-broadcast add 33.3 -> 36.8, the rest unchanged)

// ---- operations -----------------------------------------------------------------------------
struct Add { static constexpr bool binary = true; static __device__ __forceinline__ float apply(float a, float b) { return a + b; } };
struct Sub { static constexpr bool binary = true; static __device__ __forceinline__ float apply(float a, float b) { return a - b; } };
struct Mul { static constexpr bool binary = true; static __device__ __forceinline__ float apply(float a, float b) { return a * b; } };
struct Div { static constexpr bool binary = true; static __device__ __forceinline__ float apply(float a, float b) { return a / b; } };
struct Max { static constexpr bool binary = true; static __device__ __forceinline__ float apply(float a, float b) { return a >= b ? a : b; } };
struct Min { static constexpr bool binary = true; static __device__ __forceinline__ float apply(float a, float b) { return a <= b ? a : b; } };
struct Neg { static constexpr bool binary = false; static __device__ __forceinline__ float apply(float a, float) { return -a; } };
struct Exp { static constexpr bool binary = false; static __device__ __forceinline__ float apply(float a, float) { return expf(a); } };
struct Sigmoid { static constexpr bool binary = false; static __device__ __forceinline__ float apply(float a, float) { return 1.0f / (1.0f + expf(-a)); } };
struct Tanh { static constexpr bool binary = false; static __device__ __forceinline__ float apply(float a, float) { return tanhf(a); } };
// For 16-bit results the hardware exponential (a few fp32 ulps) is exact enough by a wide margin:
// its error is 2^-13 of a half / 2^-16 of a bfloat16 rounding step.  fp32 results keep libm.
struct ExpFast { static constexpr bool binary = false; static __device__ __forceinline__ float apply(float a, float) { return __expf(a); } };
struct SigmoidFast {
  static constexpr bool binary = false;
  static __device__ __forceinline__ float apply(float a, float) { return __fdividef(1.0f, 1.0f + __expf(-a)); }
};
struct TanhFast {
  static constexpr bool binary = false;
  // a quotient of two short polynomials, exact to a fraction of a 16-bit rounding step and uniformly so down to
  // the smallest arguments (see activation16_ct)
  static __device__ __forceinline__ float apply(float a, float) { return srt::activation16_ct<srtActivationTanh>(0.0f, a); }
};
struct Copy { static constexpr bool binary = false; static __device__ __forceinline__ float apply(float a, float) { return a; } };

enum OpCode { kAdd, kSub, kMul, kDiv, kMax, kMin, kNeg, kExp, kSigmoid, kTanh, kCopy };

// ---- the index space --------------------------------------------------------------------------
struct Map {
  int rank;                      // 1..MAX_RANK, innermost dimension last
  uint32_t shape[MAX_RANK];      // innermost extent counted in vectors of V elements
  long long sa[MAX_RANK], sb[MAX_RANK], so[MAX_RANK];   // element strides (innermost: per element)
  unsigned long long total;      // number of vectors
  const void* a;
  const void* b;                 // null for unary operations and for tensor-element forms
  void* o;
  float element;                 // the scalar of tensor-element forms (and of fill)
  int b_is_element;
  int fill;                      // no input at all: out = element
  int b_reused;                  // the second operand is broadcast along some dimension: its lines are read again and again
};

template <typename T, int V>
struct alignas(V * sizeof(typename T::storage)) Pack {
  typename T::storage v[V];
};

// One vector of an input operand.  STREAM: with the non-temporal hint -- an element-wise operand
// is read once, and without the hint its lines stay in L2 until evicted (the same hint raised a
// bare streaming read of this device from 5.7 to 6.2 TB/s).  A broadcast operand (a bias row under
// every row of the other operand) is the opposite case: its few lines are wanted in the caches.
template <typename T, int V, bool STREAM>
__device__ __forceinline__ Pack<T, V> load_pack(const typename T::storage* p) {
  constexpr int BYTES = V * (int)sizeof(typename T::storage);
  if constexpr (BYTES >= 8) {
    typedef uint32_t words_t __attribute__((ext_vector_type(BYTES / 4)));
    const words_t w = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const words_t*>(p))
                             : *reinterpret_cast<const words_t*>(p);
    return __builtin_bit_cast(Pack<T, V>, w);
  } else {
    return *reinterpret_cast<const Pack<T, V>*>(p);
  }
}

template <typename TI, typename TO, typename Op, int V, bool B_CACHED = false>
__global__ __launch_bounds__(256) void map_kernel(Map m) {
  using SI = typename TI::storage;
  using SO = typename TO::storage;
  const SI* a = (const SI*)m.a;
  const SI* b = (const SI*)m.b;
  SO* o = (SO*)m.o;
  const int inner = m.rank - 1;
  // four vectors per lane, a block apart, one after the other: few registers (36), eight waves per SIMD.  On
  // this device the memory parallelism of a streaming kernel comes from the waves: the same kernel with all
  // four vectors' loads issued before the first use needs 92 registers (five waves) and ran 15-20 % slower,
  // and four consecutive rows per lane with a row-broadcast operand loaded once were no faster either.
  const unsigned long long base = (unsigned long long)blockIdx.x * (256 * kVectorsPerLane) + threadIdx.x;
#pragma unroll
  for (int u = 0; u < kVectorsPerLane; ++u) {
    const unsigned long long id = base + (unsigned long long)u * 256;
    if (id >= m.total) break;
    // decompose the vector id over the collapsed dimensions
    uint32_t rest = (uint32_t)id;
    long long oa = 0, ob = 0, oo = 0;
#pragma unroll
    for (int d = MAX_RANK - 1; d >= 0; --d) {
      if (d > inner) continue;
      uint32_t idx;
      if (d == 0) {
        idx = rest;
      } else {
        const uint32_t q = rest / m.shape[d];
        idx = rest - q * m.shape[d];
        rest = q;
      }
      const long long scale = (d == inner) ? V : 1;
      oa += (long long)idx * m.sa[d] * scale;
      ob += (long long)idx * m.sb[d] * scale;
      oo += (long long)idx * m.so[d] * scale;
    }
    float fa[V], fb[V];
    if (m.fill) {
#pragma unroll
      for (int i = 0; i < V; ++i) fa[i] = m.element;
    } else if (V > 1 && m.sa[inner] == 1) {
      const Pack<TI, V> pa = load_pack<TI, V, true>(a + oa);
#pragma unroll
      for (int i = 0; i < V; ++i) fa[i] = TI::to_float(pa.v[i]);
    } else {
      // V == 1, or a broadcast along the innermost dimension
#pragma unroll
      for (int i = 0; i < V; ++i) fa[i] = TI::to_float(a[oa + (long long)i * m.sa[inner]]);
    }
    if (m.b_is_element) {
#pragma unroll
      for (int i = 0; i < V; ++i) fb[i] = m.element;
    } else if (b == nullptr) {
#pragma unroll
      for (int i = 0; i < V; ++i) fb[i] = 0.0f;
    } else if (V > 1 && m.sb[inner] == 1) {
      const Pack<TI, V> pb = load_pack<TI, V, !B_CACHED>(b + ob);
#pragma unroll
      for (int i = 0; i < V; ++i) fb[i] = TI::to_float(pb.v[i]);
    } else {
#pragma unroll
      for (int i = 0; i < V; ++i) fb[i] = TI::to_float(b[ob + (long long)i * m.sb[inner]]);
    }
    if constexpr (V > 1 && TO::dtype == srtReal16BF) {
      float r[V];
#pragma unroll
      for (int i = 0; i < V; ++i) r[i] = Op::apply(fa[i], fb[i]);
      uint32_t w[V / 2];
      encode_bf16<V>(r, w);
      *reinterpret_cast<Pack<TO, V>*>(o + oo) = __builtin_bit_cast(Pack<TO, V>, w);
    } else if (V > 1) {
      Pack<TO, V> po;
#pragma unroll
      for (int i = 0; i < V; ++i) po.v[i] = TO::from_float(Op::apply(fa[i], fb[i]));
      *reinterpret_cast<Pack<TO, V>*>(o + oo) = po;
    } else {
      o[oo] = TO::from_float(Op::apply(fa[0], fb[0]));
    }
  }
}

template <typename TI, typename TO, typename Op, int V>
hipError_t launch_v(const Map& m, hipStream_t stream) {
  const unsigned long long blocks = (m.total + 256 * kVectorsPerLane - 1) / (256 * kVectorsPerLane);
  if (blocks == 0) return hipSuccess;
  if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
  // (a run-time choice between the two kinds of load inside one kernel cost every operation 14 %)
  if constexpr (V > 1 && Op::binary) {
    if (m.b_reused) {
      hipLaunchKernelGGL((map_kernel<TI, TO, Op, V, true>), dim3((unsigned)blocks), dim3(256), 0, stream, m);
      return launch_status(stream);
    }
  }
  hipLaunchKernelGGL((map_kernel<TI, TO, Op, V>), dim3((unsigned)blocks), dim3(256), 0, stream, m);
  return launch_status(stream);
}

// Vector width the layout allows: the innermost dimension must be contiguous in the result and
// contiguous or broadcast in the inputs, its extent and every other stride of a vector-accessed
// operand a multiple of V, and the base pointers aligned to the vector.
template <typename TI, typename TO>
int vector_width(const Map& m) {
  constexpr int V = 16 / (sizeof(typename TI::storage) > sizeof(typename TO::storage) ? sizeof(typename TI::storage)
                                                                                      : sizeof(typename TO::storage));
  const int inner = m.rank - 1;
  if (m.so[inner] != 1 || m.shape[inner] % V) return 1;
  auto operand_ok = [&](const void* p, const long long* s, size_t esize, bool is_out) {
    if (!p) return true;
    if (s[inner] != 1 && (is_out || s[inner] != 0)) return false;
    if (s[inner] == 1) {
      if ((uintptr_t)p % (V * esize)) return false;
      for (int d = 0; d < inner; ++d)
        if (s[d] % V) return false;
    }
    return true;
  };
  if (!operand_ok(m.o, m.so, sizeof(typename TO::storage), true)) return 1;
  if (!m.fill && !operand_ok(m.a, m.sa, sizeof(typename TI::storage), false)) return 1;
  if (!m.fill && !m.b_is_element && !operand_ok(m.b, m.sb, sizeof(typename TI::storage), false)) return 1;
  return V;
}

template <typename TI, typename TO, typename Op>
hipError_t launch_t(Map m, hipStream_t stream) {
  constexpr int V = 16 / (sizeof(typename TI::storage) > sizeof(typename TO::storage) ? sizeof(typename TI::storage)
                                                                                      : sizeof(typename TO::storage));
  if (vector_width<TI, TO>(m) == V) {
    const int inner = m.rank - 1;
    m.shape[inner] /= V;
    m.total /= V;
    return launch_v<TI, TO, Op, V>(m, stream);
  }
  return launch_v<TI, TO, Op, 1>(m, stream);
}

template <typename Op>
hipError_t launch_same_type(int dtype, const Map& m, hipStream_t stream) {
  switch (dtype) {
    case srtReal32F: return launch_t<F32, F32, Op>(m, stream);
    case srtReal16F: return launch_t<F16, F16, Op>(m, stream);
    case srtReal16BF: return launch_t<BF16, BF16, Op>(m, stream);
    default: return hipErrorNotSupported;
  }
}

hipError_t launch_op(int op, int dtype, const Map& m, hipStream_t stream) {
  switch (op) {
    case kAdd: return launch_same_type<Add>(dtype, m, stream);
    case kSub: return launch_same_type<Sub>(dtype, m, stream);
    case kMul: return launch_same_type<Mul>(dtype, m, stream);
    case kDiv: return launch_same_type<Div>(dtype, m, stream);
    case kMax: return launch_same_type<Max>(dtype, m, stream);
    case kMin: return launch_same_type<Min>(dtype, m, stream);
    case kNeg: return launch_same_type<Neg>(dtype, m, stream);
    case kExp: return dtype == srtReal32F ? launch_same_type<Exp>(dtype, m, stream)
                                          : launch_same_type<ExpFast>(dtype, m, stream);
    case kSigmoid: return dtype == srtReal32F ? launch_same_type<Sigmoid>(dtype, m, stream)
                                              : launch_same_type<SigmoidFast>(dtype, m, stream);
    case kTanh: return dtype == srtReal32F ? launch_same_type<Tanh>(dtype, m, stream)
                                           : launch_same_type<TanhFast>(dtype, m, stream);
    case kCopy: return launch_same_type<Copy>(dtype, m, stream);
    default: return hipErrorNotSupported;
  }
}

hipError_t launch_convert(int itype, int otype, const Map& m, hipStream_t stream) {
  if (itype == otype) return launch_same_type<Copy>(itype, m, stream);
  if (itype == srtReal32F && otype == srtReal16BF) return launch_t<F32, BF16, Copy>(m, stream);
  if (itype == srtReal32F && otype == srtReal16F) return launch_t<F32, F16, Copy>(m, stream);
  if (itype == srtReal16BF && otype == srtReal32F) return launch_t<BF16, F32, Copy>(m, stream);
  if (itype == srtReal16F && otype == srtReal32F) return launch_t<F16, F32, Copy>(m, stream);
  if (itype == srtReal16BF && otype == srtReal16F) return launch_t<BF16, F16, Copy>(m, stream);
  if (itype == srtReal16F && otype == srtReal16BF) return launch_t<F16, BF16, Copy>(m, stream);
  return hipErrorNotSupported;
}

// ---- host side: descriptors -> collapsed index space -------------------------------------------
bool float_type(srtDataType t) { return t == srtReal32F || t == srtReal16F || t == srtReal16BF; }

bool desc_ok(const srtTensorDescriptor* d) { return d && d->shape && d->strides && d->rank >= 1; }

// Reads one element of `type` from host memory as fp32 (the scalar of tensor-element forms).
float host_element(srtDataType type, const void* p) {
  if (type == srtReal32F) {
    float f;
    memcpy(&f, p, 4);
    return f;
  }
  uint16_t h;
  memcpy(&h, p, 2);
  if (type == srtReal16BF) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
  }
  _Float16 x;
  memcpy(&x, &h, 2);
  return (float)x;
}

// Builds the index space of `out` with the strides of each operand, dropping extent-1
// dimensions and merging neighbours that every operand walks contiguously (or broadcasts).
// Returns srtErrorNotSupported when more than MAX_RANK dimensions remain.
srtStatus build_map(const srtTensorDescriptor* ad, const srtTensorDescriptor* bd, const srtTensorDescriptor* od,
                    Map* m, bool* empty) {
  *empty = false;
  const uint32_t rank = od->rank;
  if (rank > 8) return srtErrorNotSupported;
  if ((ad && ad->rank != rank) || (bd && bd->rank != rank)) return srtErrorInvalidValue;
  size_t shape[8];
  long long sa[8], sb[8], so[8];
  int n = 0;
  unsigned long long total = 1;
  for (uint32_t d = 0; d < rank; ++d) {
    const size_t e = od->shape[d];
    if ((ad && ad->shape[d] != e) || (bd && bd->shape[d] != e)) return srtErrorInvalidValue;
    total *= e;
    if (e == 1) continue;
    shape[n] = e;
    sa[n] = ad ? (long long)ad->strides[d] : 0;
    sb[n] = bd ? (long long)bd->strides[d] : 0;
    so[n] = (long long)od->strides[d];
    ++n;
  }
  if (total == 0) { *empty = true; return srtSuccess; }
  if (n == 0) { shape[0] = 1; sa[0] = sb[0] = 0; so[0] = 1; n = 1; }
  // merge d into d + 1 where stride[d] == shape[d + 1] * stride[d + 1] for every operand
  int w = 0;
  for (int d = 1; d < n; ++d) {
    const long long e = (long long)shape[d];
    if (sa[w] == e * sa[d] && sb[w] == e * sb[d] && so[w] == e * so[d]) {
      shape[w] *= shape[d];
      sa[w] = sa[d]; sb[w] = sb[d]; so[w] = so[d];
    } else {
      ++w;
      shape[w] = shape[d]; sa[w] = sa[d]; sb[w] = sb[d]; so[w] = so[d];
    }
  }
  n = w + 1;
  if (n > MAX_RANK) return srtErrorNotSupported;
  m->rank = n;
  for (int d = 0; d < MAX_RANK; ++d) {
    m->shape[d] = 1; m->sa[d] = m->sb[d] = m->so[d] = 0;
  }
  for (int d = 0; d < n; ++d) {
    if (shape[d] > 0xffffffffull) return srtErrorNotSupported;
    m->shape[d] = (uint32_t)shape[d];
    m->sa[d] = sa[d]; m->sb[d] = sb[d]; m->so[d] = so[d];
  }
  if (total > 0xffffffffull) return srtErrorNotSupported;   // the kernel decomposes 32-bit ids
  m->total = total;
  m->b_reused = 0;
  for (int d = 0; d < n; ++d)
    if (bd && shape[d] > 1 && sb[d] == 0) m->b_reused = 1;
  return srtSuccess;
}

srtStatus binary(int op, const void* a, const srtTensorDescriptor* ad, const void* b, const srtTensorDescriptor* bd,
                 void* out, const srtTensorDescriptor* od, srtStream stream) {
  if (!desc_ok(ad) || !desc_ok(bd) || !desc_ok(od)) return srtErrorInvalidValue;
  if (!float_type(od->type) || ad->type != od->type || bd->type != od->type) return srtErrorNotSupported;
  Map m{};
  bool empty;
  srtStatus s = build_map(ad, bd, od, &m, &empty);
  if (s != srtSuccess || empty) return s;
  if (!a || !b || !out) return srtErrorInvalidValue;
  m.a = a; m.b = b; m.o = out;
  return from_hip(launch_op(op, od->type, m, reinterpret_cast<hipStream_t>(stream)));
}

srtStatus binary_element(int op, const void* a, const srtTensorDescriptor* ad, const void* element, void* out,
                         const srtTensorDescriptor* od, srtStream stream) {
  if (!desc_ok(ad) || !desc_ok(od) || !element) return srtErrorInvalidValue;
  if (!float_type(od->type) || ad->type != od->type) return srtErrorNotSupported;
  Map m{};
  bool empty;
  srtStatus s = build_map(ad, nullptr, od, &m, &empty);
  if (s != srtSuccess || empty) return s;
  if (!a || !out) return srtErrorInvalidValue;
  m.a = a; m.o = out;
  m.b_is_element = 1;
  m.element = host_element(od->type, element);
  return from_hip(launch_op(op, od->type, m, reinterpret_cast<hipStream_t>(stream)));
}

srtStatus unary(int op, const void* a, const srtTensorDescriptor* ad, void* out, const srtTensorDescriptor* od,
                srtStream stream) {
  if (!desc_ok(ad) || !desc_ok(od)) return srtErrorInvalidValue;
  if (!float_type(od->type) || !float_type(ad->type)) return srtErrorNotSupported;
  if (op != kCopy && ad->type != od->type) return srtErrorNotSupported;
  Map m{};
  bool empty;
  srtStatus s = build_map(ad, nullptr, od, &m, &empty);
  if (s != srtSuccess || empty) return s;
  if (!a || !out) return srtErrorInvalidValue;
  m.a = a; m.o = out;
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  if (op == kCopy) return from_hip(launch_convert(ad->type, od->type, m, hs));
  return from_hip(launch_op(op, od->type, m, hs));
}

void flat_map(size_t count, Map* m) {
  m->rank = 1;
  for (int d = 0; d < MAX_RANK; ++d) { m->shape[d] = 1; m->sa[d] = m->sb[d] = m->so[d] = 0; }
  m->sa[0] = m->sb[0] = m->so[0] = 1;
  m->total = count;
}

// Flat forms take a count, not a descriptor.  Long buffers are cut into pieces the 32-bit innermost
// extent can hold, and a count that is not a multiple of the vector width into a vector body and a
// short element-wise tail (the buffers themselves are allocation-aligned).
template <typename F>
srtStatus flat_pieces(size_t count, size_t in_size, size_t out_size, Map m, F launch) {
  const size_t piece = (size_t)1 << 30;
  size_t done = 0;
  while (done < count) {
    size_t n = count - done < piece ? count - done : piece;
    if (n > 8 && n % 8) n -= n % 8;   // body now, tail in the next round
    Map p = m;
    flat_map(n, &p);
    p.shape[0] = (uint32_t)n;
    if (m.a) p.a = (const char*)m.a + done * in_size;
    if (m.b) p.b = (const char*)m.b + done * in_size;
    p.o = (char*)m.o + done * out_size;
    srtStatus s = from_hip(launch(p));
    if (s != srtSuccess) return s;
    done += n;
  }
  return srtSuccess;
}

size_t type_size(srtDataType t) { return t == srtReal32F ? 4 : 2; }

}  // namespace ew
}  // namespace srt

using namespace srt::ew;

extern "C" {

#define SRT_BINARY(Name, code)                                                                              \
  srtStatus srt##Name(const void* a, const srtTensorDescriptor* aDesc, const void* b,                        \
                      const srtTensorDescriptor* bDesc, void* out, const srtTensorDescriptor* oDesc,         \
                      srtStream stream) {                                                                    \
    return binary(code, a, aDesc, b, bDesc, out, oDesc, stream);                                            \
  }                                                                                                          \
  srtStatus srt##Name##TE(const void* a, const srtTensorDescriptor* aDesc, const void* element, void* out,   \
                          const srtTensorDescriptor* oDesc, srtStream stream) {                              \
    return binary_element(code, a, aDesc, element, out, oDesc, stream);                                     \
  }

SRT_BINARY(Add, kAdd)
SRT_BINARY(Sub, kSub)
SRT_BINARY(Mul, kMul)
SRT_BINARY(Div, kDiv)
SRT_BINARY(Max, kMax)
SRT_BINARY(Min, kMin)

#define SRT_UNARY(Name, code)                                                                     \
  srtStatus srt##Name(const void* a, const srtTensorDescriptor* aDesc, void* out,                  \
                      const srtTensorDescriptor* oDesc, srtStream stream) {                        \
    return unary(code, a, aDesc, out, oDesc, stream);                                             \
  }

SRT_UNARY(Neg, kNeg)
SRT_UNARY(Exp, kExp)
SRT_UNARY(Sigmoid, kSigmoid)
SRT_UNARY(Tanh, kTanh)
SRT_UNARY(Copy, kCopy)

// Dense tensor-tensor and tensor-element forms of the six binary operators: what CudaQueue calls when
// canFlatten holds (Sources/SwiftRTCore/platform/cuda/functions/CudaMath.swift:103-113).
static srtStatus binary_flat(int op, srtDataType type, const void* a, const void* b, const void* element, void* out,
                             size_t count, srtStream stream) {
  if (!float_type(type)) return srtErrorNotSupported;
  if (count == 0) return srtSuccess;
  if (!a || !out || (!b && !element)) return srtErrorInvalidValue;
  Map m{};
  m.a = a; m.b = b; m.o = out;
  if (!b) {
    m.b_is_element = 1;
    m.element = host_element(type, element);
  }
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  return flat_pieces(count, type_size(type), type_size(type), m,
                     [&](const Map& p) { return launch_op(op, type, p, hs); });
}

#define SRT_BINARY_FLAT(Name, code)                                                                          \
  srtStatus srt##Name##Flat(srtDataType type, const void* a, const void* b, void* out, size_t count,          \
                            srtStream stream) {                                                               \
    return binary_flat(code, type, a, b, nullptr, out, count, stream);                                       \
  }                                                                                                           \
  srtStatus srt##Name##TEFlat(const void* a, srtDataType atype, const void* element, void* out, size_t count, \
                              srtStream stream) {                                                             \
    return binary_flat(code, atype, a, nullptr, element, out, count, stream);                                \
  }

SRT_BINARY_FLAT(Add, kAdd)
SRT_BINARY_FLAT(Sub, kSub)
SRT_BINARY_FLAT(Mul, kMul)
SRT_BINARY_FLAT(Div, kDiv)
SRT_BINARY_FLAT(Max, kMax)
SRT_BINARY_FLAT(Min, kMin)

// the reference spells the comparison family's tensor-element form the other way round, with the type first
srtStatus srtMinFlatTE(srtDataType type, const void* a, const void* element, void* out, size_t count, srtStream stream) {
  return binary_flat(kMin, type, a, nullptr, element, out, count, stream);
}
srtStatus srtMaxFlatTE(srtDataType type, const void* a, const void* element, void* out, size_t count, srtStream stream) {
  return binary_flat(kMax, type, a, nullptr, element, out, count, stream);
}

srtStatus srtCopyFlat(srtDataType atype, const void* a, srtDataType otype, void* out, size_t count,
                      srtStream stream) {
  if (!float_type(atype) || !float_type(otype)) return srtErrorNotSupported;
  if (count == 0) return srtSuccess;
  if (!a || !out) return srtErrorInvalidValue;
  Map m{};
  m.a = a; m.o = out;
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  return flat_pieces(count, type_size(atype), type_size(otype), m,
                     [&](const Map& p) { return launch_convert(atype, otype, p, hs); });
}

srtStatus srtFillFlat(srtDataType type, void* out, const void* element, size_t count, srtStream stream) {
  if (!float_type(type)) return srtErrorNotSupported;
  if (count == 0) return srtSuccess;
  if (!out || !element) return srtErrorInvalidValue;
  Map m{};
  m.o = out;
  m.fill = 1;
  m.element = host_element(type, element);
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  return flat_pieces(count, type_size(type), type_size(type), m,
                     [&](const Map& p) { return launch_op(kCopy, type, p, hs); });
}

}  // extern "C"
