/*
 * srt_oracle.c -- CPU restatement of SwiftRT's matmul path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker for the HIP library, never the product: only the test suite,
 * the smoke check and the benchmark's cpu_baseline leg may load it.  Nothing in the
 * shipped library links, loads or calls it.
 *
 * Every function cites the reference source it restates (paths relative to the
 * reference checkout).  The reference is Swift and cannot be built in this environment
 * (no Swift toolchain), so these are restatements, pinned by:
 *   - the reference's own known-answer tests (3x2 . 2x4 matmul and its commented gradient /
 *     batched expectations, the LSTM fixtures that pin matmul + bias + sigmoid/tanh),
 *   - library oracles (numpy float16, numpy float64 matmul),
 *   - closed forms and brute force (exhaustive bf16 rounding sweep against an independent
 *     formula, integer-valued inputs that are exact in every order).
 * Parity status per function is stated in its comment.  Two facts only a Swift run could
 * confirm are marked "restated, unconfirmed".
 *
 * Build: gcc -O2 -ffp-contract=off -fopenmp -shared -fPIC (see Makefile).  -ffp-contract=off
 * matters: the reference multiplies then adds (Swift never fuses implicitly).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

/* element type ids: numeric values match the library's srtDataType */
enum { ORA_F32 = 0, ORA_F16 = 2, ORA_BF16 = 14 };

/* accumulator choice for the restated dot product */
enum {
  ORA_ACC_VALUE = 0, /* E.Value as the Linux reference has it: f32->f32, bf16->f32, f16->f16 */
  ORA_ACC_F32 = 1    /* fp32 accumulate for every type (the specification for the GPU path;
                        also what the reference does for Float16 on macOS) */
};

/* activation ids follow ActivationType's case order,
 * Sources/SwiftRTCore/platform/common/FunctionProperties.swift:44-51 */
enum { ORA_SIGMOID = 0, ORA_RELU = 1, ORA_TANH = 2, ORA_CLIPPED_RELU = 3, ORA_ELU = 4, ORA_IDENTITY = 5 };

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ---------------------------------------------------------------------------------------
 * BFloat16 codec.
 * Follows Sources/SwiftRTCore/platform/common/BFloat16.swift:53-80 (float2bfloat16_rn and
 * float2bfloat16): NaN -> 0x7FFF, otherwise truncate to the high 16 bits and round up when
 * the dropped 16 bits, taken as a 32-bit remainder (x << 16), exceed 0x80000000, or equal
 * it with an odd kept value (round to nearest, ties to even).
 * Parity: pinned (exhaustive 2^32 sweep against an independent formula; bf16 add KAT).
 * ------------------------------------------------------------------------------------- */
ORACLE_API uint16_t srt_oracle_f32_to_bf16(float f) {
  uint32_t x = f32_bits(f);
  uint16_t raw;
  uint32_t rem;
  if ((x & 0x7fffffffu) > 0x7f800000u) {
    rem = 0;
    raw = 0x7fff;
  } else {
    rem = x << 16;
    raw = (uint16_t)(x >> 16);
  }
  if (rem > 0x80000000u || (rem == 0x80000000u && (raw & 1u))) raw = (uint16_t)(raw + 1);
  return raw;
}

/* BFloat16.swift:83-85: bfloat162float = bits << 16 */
ORACLE_API float srt_oracle_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* ---------------------------------------------------------------------------------------
 * Float16 codec (IEEE binary16, round to nearest even).
 * On Linux the reference uses the native Float16 (Float16.swift:12-16); its macOS
 * emulation (Float16.swift:54-134) is the same IEEE RNE conversion.  Written from the
 * IEEE definition.  Parity: pinned against numpy.float16 (all 65536 decodes, encode of
 * every bf16-exact and many random floats including ties, subnormals, overflow).
 * ------------------------------------------------------------------------------------- */
ORACLE_API float srt_oracle_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  if (exp == 0x1f) return bits_f32(sign | 0x7f800000u | (man << 13)); /* inf / nan */
  if (exp == 0) {
    if (man == 0) return bits_f32(sign);
    /* subnormal: value = man * 2^-24 */
    float v = (float)man * 5.9604644775390625e-08f;
    return bits_f32(f32_bits(v) | sign);
  }
  return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

ORACLE_API uint16_t srt_oracle_f32_to_f16(float f) {
  uint32_t x = f32_bits(f);
  uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  uint32_t u = x & 0x7fffffffu;
  if (u > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((u >> 13) & 0x3ffu)); /* nan (quiet) */
  if (u >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 rounds to inf */
  if (u < 0x33000001u) return sign;                         /* <= 2^-25 rounds to zero */
  int32_t e = (int32_t)(u >> 23) - 127;
  uint32_t m = (u & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  uint32_t shift, half_exp;
  if (e < -14) { /* result is subnormal: value = m * 2^(e-23); unit = 2^-24 */
    shift = (uint32_t)(13 + (-14 - e));
    half_exp = 0;
  } else {
    shift = 13;
    half_exp = (uint32_t)(e + 15);
  }
  uint32_t kept = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (kept & 1u))) kept++;
  /* normal: kept includes the hidden bit (0x400); adding it to the exponent field carries
   * correctly when rounding overflows the mantissa.  subnormal: kept is the raw field and
   * a carry into 0x400 yields the smallest normal, which is also right. */
  uint32_t out = (half_exp == 0) ? kept : (((half_exp - 1u) << 10) + kept);
  return (uint16_t)(sign | out);
}

/* load one element as its Value type widened to float */
static inline float load_elem(int dtype, const void* p, int64_t i) {
  switch (dtype) {
    case ORA_F32: return ((const float*)p)[i];
    case ORA_F16: return srt_oracle_f16_to_f32(((const uint16_t*)p)[i]);
    default: return srt_oracle_bf16_to_f32(((const uint16_t*)p)[i]);
  }
}

static inline void store_elem(int dtype, void* p, int64_t i, float v) {
  switch (dtype) {
    case ORA_F32: ((float*)p)[i] = v; break;
    case ORA_F16: ((uint16_t*)p)[i] = srt_oracle_f32_to_f16(v); break;
    default: ((uint16_t*)p)[i] = srt_oracle_f32_to_bf16(v); break;
  }
}

static inline float round_to_f16(float v) { return srt_oracle_f16_to_f32(srt_oracle_f32_to_f16(v)); }

ORACLE_API int srt_oracle_elem_size(int dtype) {
  return dtype == ORA_F32 ? 4 : (dtype == ORA_F16 || dtype == ORA_BF16) ? 2 : 0;
}

/* ---------------------------------------------------------------------------------------
 * cpu_matmul, rank 2 and rank 3.
 * Follows Sources/SwiftRTCore/platform/cpu/functions/CpuMath.swift:1141-1161 (rank 2) and
 * :1164-1186 (rank 3):
 *   lhs = transposeLhs ? lhs.t : lhs      -- .t swaps the last two extents AND strides,
 *   rhs = transposeRhs ? rhs.t : rhs         zero copy (tensor/TensorInit.swift:844-890,
 *                                            tensor/Shape.swift:208-212)
 *   for r, for c: out[r, c] = zip(row r of lhs, column c of rhs).reduce(0) { $0 += a * b }
 * i.e. k ascending, a separate multiply and add per term, accumulator of type E.Value,
 * converted to the stored type once at the end (E.store).
 *
 * `rank` is 2 or 3; shapes/strides are in elements, as stored (before any transpose), with
 * the batch extent first for rank 3.  For Float16 with ORA_ACC_VALUE every product and
 * every sum is rounded to binary16, which is what native Float16 arithmetic does (computed
 * here in float and rounded: exact for one +,* because 24 >= 2*11+2).
 * Returns 0, or -1 when the extents do not agree (the reference asserts).
 * Parity: pinned for f32 (reference KATs); order/precision for bf16 and f16 follow the
 * closed reading of the loop and codecs, pinned by exact integer-valued cases; bit-identity
 * with what swiftc emits is "restated, unconfirmed".
 * ------------------------------------------------------------------------------------- */
ORACLE_API int srt_oracle_matmul(int dtype, int acc_mode, int rank,
                                 const void* lhs, const int64_t* lhs_shape, const int64_t* lhs_strides,
                                 int transpose_lhs,
                                 const void* rhs, const int64_t* rhs_shape, const int64_t* rhs_strides,
                                 int transpose_rhs,
                                 void* out, const int64_t* out_shape, const int64_t* out_strides) {
  if (rank != 2 && rank != 3) return -1;
  if (!srt_oracle_elem_size(dtype)) return -1;
  const int b = rank - 2; /* index of the row extent */
  int64_t ls[3], lst[3], rs[3], rst[3];
  for (int i = 0; i < rank; ++i) {
    ls[i] = lhs_shape[i]; lst[i] = lhs_strides[i];
    rs[i] = rhs_shape[i]; rst[i] = rhs_strides[i];
  }
  if (transpose_lhs) {
    int64_t t = ls[b]; ls[b] = ls[b + 1]; ls[b + 1] = t;
    t = lst[b]; lst[b] = lst[b + 1]; lst[b + 1] = t;
  }
  if (transpose_rhs) {
    int64_t t = rs[b]; rs[b] = rs[b + 1]; rs[b + 1] = t;
    t = rst[b]; rst[b] = rst[b + 1]; rst[b + 1] = t;
  }
  const int64_t M = out_shape[b], N = out_shape[b + 1], K = ls[b + 1];
  if (ls[b] != M || rs[b + 1] != N || rs[b] != K) return -1;
  const int64_t batch = rank == 3 ? out_shape[0] : 1;
  if (rank == 3 && (ls[0] != batch || rs[0] != batch)) return -1;
  const int f16_value_acc = (dtype == ORA_F16 && acc_mode == ORA_ACC_VALUE);

  for (int64_t n = 0; n < batch; ++n) {
    const int64_t lb = rank == 3 ? n * lst[0] : 0;
    const int64_t rb = rank == 3 ? n * rst[0] : 0;
    const int64_t ob = rank == 3 ? n * out_strides[0] : 0;
    for (int64_t r = 0; r < M; ++r) {
      for (int64_t c = 0; c < N; ++c) {
        float acc = 0.0f;
        if (f16_value_acc) {
          for (int64_t k = 0; k < K; ++k) {
            float a = load_elem(dtype, lhs, lb + r * lst[b] + k * lst[b + 1]);
            float w = load_elem(dtype, rhs, rb + k * rst[b] + c * rst[b + 1]);
            float p = round_to_f16(a * w);
            acc = round_to_f16(acc + p);
          }
        } else {
          for (int64_t k = 0; k < K; ++k) {
            float a = load_elem(dtype, lhs, lb + r * lst[b] + k * lst[b + 1]);
            float w = load_elem(dtype, rhs, rb + k * rst[b] + c * rst[b + 1]);
            float p = a * w;
            acc += p;
          }
        }
        store_elem(dtype, out, ob + r * out_strides[b] + c * out_strides[b + 1], acc);
      }
    }
  }
  return 0;
}

/* ---------------------------------------------------------------------------------------
 * Activation functions on E.Value (float here).
 *   sigmoid: 1 / (1 + exp(-x))                 CpuMath.swift:1369-1377
 *   tanh:    libm tanh                         CpuMath.swift (cpu_tanh -> .tanh)
 *   relu:    max(x, 0)                         no reference function exists; the shape is
 *                                              max(tensor, scalar), test_Comparative.swift:214-218
 *   clippedRelu: min(max(x,0), coef)           ceiling = activationReluCeiling,
 *                                              CpuConvolution.swift:23,34 (cuDNN definition)
 *   elu:     x > 0 ? x : coef * (exp(x) - 1)   cuDNN definition (coef = alpha); the reference
 *                                              only forwards the enum to cuDNN
 *   identity
 * Parity: sigmoid and tanh pinned by the LSTM fixtures; relu/clippedRelu/elu are closed
 * forms ("parity unpinned" against the reference: it has no implementation to compare).
 * ------------------------------------------------------------------------------------- */
ORACLE_API float srt_oracle_activation(int activation, float coef, float x) {
  switch (activation) {
    case ORA_SIGMOID: return 1.0f / (1.0f + expf(-x));
    case ORA_RELU: return x > 0.0f ? x : 0.0f;
    case ORA_TANH: return tanhf(x);
    case ORA_CLIPPED_RELU: { float y = x > 0.0f ? x : 0.0f; return y < coef ? y : coef; }
    case ORA_ELU: return x > 0.0f ? x : coef * (expf(x) - 1.0f);
    default: return x;
  }
}

/* ---------------------------------------------------------------------------------------
 * Dense forward:  y = activation(matmul(x, W) + bias), rank 2, bias broadcast over rows.
 * The reference's Dense.callAsFunction is a stub (SwiftRTLayers/Dense.swift:36-39) and
 * matmul(bias:) drops its bias (operators/Matmul.swift:57-72), so the semantics are those
 * the layers in use spell out as three ops: tanh(matmul(x, W) + b)
 * (SwiftRTLayers/Recurrent.swift:157-161) and sigmoid/tanh of matmul(x, W, bias: b)
 * (Recurrent.swift:255-266).
 *   fused != 0: one rounding -- act(acc + bias) computed in float, stored once (the
 *               definition the GPU epilogue implements)
 *   fused == 0: as three reference ops would run: store matmul result to E, add bias in
 *               E.Value and store, apply the activation and store (three roundings)
 * bias may be NULL.  Parity: pinned through the LSTM fixtures (f32, where both variants
 * coincide up to the final rounding).
 * ------------------------------------------------------------------------------------- */
ORACLE_API int srt_oracle_dense_forward(int dtype, int acc_mode, int fused,
                                        const void* x, const int64_t* x_shape, const int64_t* x_strides,
                                        int transpose_x,
                                        const void* w, const int64_t* w_shape, const int64_t* w_strides,
                                        int transpose_w,
                                        const void* bias, int64_t bias_stride,
                                        int activation, float coef,
                                        void* out, const int64_t* out_shape, const int64_t* out_strides) {
  const int64_t M = out_shape[0], N = out_shape[1];
  if (!fused) {
    int rc = srt_oracle_matmul(dtype, acc_mode, 2, x, x_shape, x_strides, transpose_x, w, w_shape,
                               w_strides, transpose_w, out, out_shape, out_strides);
    if (rc) return rc;
    for (int64_t r = 0; r < M; ++r)
      for (int64_t c = 0; c < N; ++c) {
        int64_t o = r * out_strides[0] + c * out_strides[1];
        float v = load_elem(dtype, out, o);
        if (bias) {
          float s = v + load_elem(dtype, bias, c * bias_stride);
          if (dtype == ORA_F16 && acc_mode == ORA_ACC_VALUE) s = round_to_f16(s);
          store_elem(dtype, out, o, s);
          v = load_elem(dtype, out, o);
        }
        store_elem(dtype, out, o, srt_oracle_activation(activation, coef, v));
      }
    return 0;
  }
  /* fused: accumulate in float as cpu_matmul does for f32/bf16 (and fp32 for f16 unless the
   * caller asks for Value accumulation), then bias and activation before the single store */
  int64_t xs[2] = {x_shape[0], x_shape[1]}, xst[2] = {x_strides[0], x_strides[1]};
  int64_t ws[2] = {w_shape[0], w_shape[1]}, wst[2] = {w_strides[0], w_strides[1]};
  if (transpose_x) { int64_t t = xs[0]; xs[0] = xs[1]; xs[1] = t; t = xst[0]; xst[0] = xst[1]; xst[1] = t; }
  if (transpose_w) { int64_t t = ws[0]; ws[0] = ws[1]; ws[1] = t; t = wst[0]; wst[0] = wst[1]; wst[1] = t; }
  const int64_t K = xs[1];
  if (xs[0] != M || ws[1] != N || ws[0] != K) return -1;
  const int f16_value_acc = (dtype == ORA_F16 && acc_mode == ORA_ACC_VALUE);
  for (int64_t r = 0; r < M; ++r)
    for (int64_t c = 0; c < N; ++c) {
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k) {
        float a = load_elem(dtype, x, r * xst[0] + k * xst[1]);
        float b = load_elem(dtype, w, k * wst[0] + c * wst[1]);
        float p = a * b;
        if (f16_value_acc) { p = round_to_f16(p); acc = round_to_f16(acc + p); }
        else acc += p;
      }
      if (bias) acc = acc + load_elem(dtype, bias, c * bias_stride);
      store_elem(dtype, out, r * out_strides[0] + c * out_strides[1],
                 srt_oracle_activation(activation, coef, acc));
    }
  return 0;
}

/* ---------------------------------------------------------------------------------------
 * Grading oracle: fp64 GEMM on the already dtype-rounded inputs.  Not a restatement of a
 * reference function -- it is the yardstick the error bars are measured against
 * (max |c - c64| / max |c64|).  Computes the listed rows of op(A).op(B) (all N columns
 * each) into out64[nrows][N]; rows == NULL means rows 0..nrows-1.  Strides are in elements
 * as stored; transposes swap them as above.  OpenMP over rows.
 * Parity: pinned against numpy float64 matmul.
 * ------------------------------------------------------------------------------------- */
ORACLE_API int srt_oracle_gemm_f64_rows(int dtype,
                                        const void* lhs, const int64_t* lhs_shape, const int64_t* lhs_strides,
                                        int transpose_lhs,
                                        const void* rhs, const int64_t* rhs_shape, const int64_t* rhs_strides,
                                        int transpose_rhs,
                                        int64_t nrows, const int64_t* rows, double* out64) {
  if (!srt_oracle_elem_size(dtype)) return -1;
  int64_t ls[2] = {lhs_shape[0], lhs_shape[1]}, lst[2] = {lhs_strides[0], lhs_strides[1]};
  int64_t rs[2] = {rhs_shape[0], rhs_shape[1]}, rst[2] = {rhs_strides[0], rhs_strides[1]};
  if (transpose_lhs) { int64_t t = ls[0]; ls[0] = ls[1]; ls[1] = t; t = lst[0]; lst[0] = lst[1]; lst[1] = t; }
  if (transpose_rhs) { int64_t t = rs[0]; rs[0] = rs[1]; rs[1] = t; t = rst[0]; rst[0] = rst[1]; rst[1] = t; }
  const int64_t M = ls[0], K = ls[1], N = rs[1];
  if (rs[0] != K) return -1;
  /* widen B once to a dense K x N double panel so the inner loop streams contiguously */
  double* bd = (double*)malloc((size_t)K * (size_t)N * sizeof(double));
  if (!bd) return -2;
#pragma omp parallel for schedule(static)
  for (int64_t k = 0; k < K; ++k)
    for (int64_t c = 0; c < N; ++c) bd[k * N + c] = (double)load_elem(dtype, rhs, k * rst[0] + c * rst[1]);
  int bad = 0;
#pragma omp parallel for schedule(dynamic, 1)
  for (int64_t i = 0; i < nrows; ++i) {
    int64_t r = rows ? rows[i] : i;
    if (r < 0 || r >= M) { bad = 1; continue; }
    double* o = out64 + i * N;
    for (int64_t c = 0; c < N; ++c) o[c] = 0.0;
    for (int64_t k = 0; k < K; ++k) {
      double a = (double)load_elem(dtype, lhs, r * lst[0] + k * lst[1]);
      const double* brow = bd + k * N;
      for (int64_t c = 0; c < N; ++c) o[c] += a * brow[c];
    }
  }
  free(bd);
  return bad ? -1 : 0;
}

/* number of threads the OpenMP loops above use */
ORACLE_API int srt_oracle_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* bulk codecs for the tests (count elements) */
ORACLE_API void srt_oracle_encode(int dtype, const float* src, void* dst, int64_t count) {
  for (int64_t i = 0; i < count; ++i) store_elem(dtype, dst, i, src[i]);
}
ORACLE_API void srt_oracle_decode(int dtype, const void* src, float* dst, int64_t count) {
  for (int64_t i = 0; i < count; ++i) dst[i] = load_elem(dtype, src, i);
}

/* Exhaustive check of the bf16 encoder against an independent statement of RNE
 * ((x + 0x7FFF + lsb) >> 16 with a NaN guard) over [first, last] bit patterns.
 * Returns the number of mismatches. */
ORACLE_API uint64_t srt_oracle_bf16_sweep(uint32_t first, uint32_t last) {
  uint64_t bad = 0;
  uint64_t a = first, b = last;
#pragma omp parallel for reduction(+ : bad) schedule(static)
  for (uint64_t x = a; x <= b; ++x) {
    uint32_t u = (uint32_t)x;
    uint16_t want;
    if ((u & 0x7fffffffu) > 0x7f800000u) want = 0x7fff;
    else want = (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
    if (srt_oracle_f32_to_bf16(bits_f32(u)) != want) bad++;
  }
  return bad;
}
