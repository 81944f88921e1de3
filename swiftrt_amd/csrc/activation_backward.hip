// Backward of the Dense epilogue: the activation gradient fused with the bias gradient.
//
//   dx[m, n]  = dy[m, n] * act'(y[m, n])          (act' written in terms of the OUTPUT y, as
//                                                  cudnnActivationBackward uses it for these modes)
//   dbias[n]  = sum_m dx[m, n]                     (fp32 sums, rounded once)
//
// The two GEMMs of the backward pass (dX = dZ . W^T, dW = X^T . dZ) are ordinary srtMatmul calls
// with transpose flags; this kernel produces their common operand dZ in ONE pass over y and dy
// and gets the bias gradient for free from the values it already holds.  Bandwidth-bound:
// algorithmic bytes = 3 M N elements (read y, dy; write dx) + N.
//
//   grid    x: strips of 64 lanes x V columns, y: row chunks; 4 waves per workgroup, wave w takes
//           rows w, w + 4, ... of its chunk, so every wave instruction moves one 1 KiB row segment
//   sums    8 (V) fp32 column sums per lane in registers, waves combined through LDS, one fp32
//           partial row per chunk in a workspace; a second tiny kernel adds the chunks in a fixed
//           order (deterministic, no atomics), eight rows in flight per lane
//   V = 1   same structure for layouts the vector path excludes (any strides)
#include "gemm_common.h"
#include "status.h"

namespace srt {
namespace {

// derivative of the activation expressed through its output
__device__ __forceinline__ float activation_slope(int activation, float coef, float y) {
  switch (activation) {
    case srtActivationSigmoid: return y * (1.0f - y);
    case srtActivationRelu: return y > 0.0f ? 1.0f : 0.0f;
    case srtActivationTanh: return 1.0f - y * y;
    case srtActivationClippedRelu: return (y > 0.0f && y < coef) ? 1.0f : 0.0f;
    case srtActivationElu: return y > 0.0f ? 1.0f : y + coef;
    default: return 1.0f;
  }
}

struct BackwardProblem {
  int M, N;
  const void* y;
  const void* dy;
  void* dx;
  long long sym, syn, sdm, sdn, sxm, sxn;   // element strides of y, dy, dx
  float* partial;                            // [chunks][N] fp32, null when no bias gradient is wanted
  int rows_per_chunk;
  int activation;
  float coef;
};

template <typename T, int V>
struct alignas(V * sizeof(typename T::storage)) Pack {
  typename T::storage v[V];
};

// One vector of y or dy, with the non-temporal hint: both are read exactly once.
template <typename T, int V>
__device__ __forceinline__ Pack<T, V> load_once(const typename T::storage* p) {
  constexpr int BYTES = V * (int)sizeof(typename T::storage);
  if constexpr (BYTES >= 8) {
    typedef uint32_t words_t __attribute__((ext_vector_type(BYTES / 4)));
    return __builtin_bit_cast(Pack<T, V>, __builtin_nontemporal_load(reinterpret_cast<const words_t*>(p)));
  } else {
    return *reinterpret_cast<const Pack<T, V>*>(p);
  }
}

template <typename T, int V, int R>
__global__ __launch_bounds__(256) void activation_backward_kernel(BackwardProblem p) {
  using S = typename T::storage;
  __shared__ float red[4][64 * V];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = (blockIdx.x * 64 + lane) * V;
  const int m_begin = blockIdx.y * p.rows_per_chunk;
  const int m_end = min(p.M, m_begin + p.rows_per_chunk);
  const S* y = (const S*)p.y;
  const S* dy = (const S*)p.dy;
  S* dx = (S*)p.dx;
  float sum[V];
#pragma unroll
  for (int i = 0; i < V; ++i) sum[i] = 0.0f;
  if (n0 < p.N) {
    // R rows per trip (all their loads are issued before any is used); a row past the chunk's end repeats
    // the trip's first row and is not stored or summed
    for (int m = m_begin + wave; m < m_end; m += 4 * R) {
      Pack<T, V> py[R], pd[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int row = m + 4 * r < m_end ? m + 4 * r : m;
        if (V > 1) {
          py[r] = load_once<T, V>(y + (long long)row * p.sym + n0);
          pd[r] = load_once<T, V>(dy + (long long)row * p.sdm + n0);
        } else {
          py[r].v[0] = y[(long long)row * p.sym + (long long)n0 * p.syn];
          pd[r].v[0] = dy[(long long)row * p.sdm + (long long)n0 * p.sdn];
        }
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int row = m + 4 * r;
        if (r > 0 && row >= m_end) break;
        Pack<T, V> out;
        float gs[V];
#pragma unroll
        for (int i = 0; i < V; ++i) {
          float g = T::to_float(pd[r].v[i]) * activation_slope(p.activation, p.coef, T::to_float(py[r].v[i]));
          // keep the product as an fp32 value: without this the compiler merges the multiply and
          // the conversion to half into one mixed-precision instruction that rounds the exact
          // product once, which differs from "fp32 product, then round" on ties
          asm volatile("" : "+v"(g));
          gs[i] = g;
          sum[i] += g;
        }
        if constexpr (V > 1 && T::dtype == srtReal16BF) {
          uint32_t w[V / 2];
          encode_bf16<V>(gs, w);
          out = __builtin_bit_cast(Pack<T, V>, w);
        } else {
#pragma unroll
          for (int i = 0; i < V; ++i) out.v[i] = T::from_float(gs[i]);
        }
        if (V > 1) *reinterpret_cast<Pack<T, V>*>(dx + (long long)row * p.sxm + n0) = out;
        else dx[(long long)row * p.sxm + (long long)n0 * p.sxn] = out.v[0];
      }
    }
  }
  if (p.partial == nullptr) return;
#pragma unroll
  for (int i = 0; i < V; ++i) red[wave][lane * V + i] = sum[i];
  __syncthreads();
  if (wave == 0 && n0 < p.N) {
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const int c = lane * V + i;
      p.partial[(long long)blockIdx.y * p.N + n0 + i] = (red[0][c] + red[1][c]) + (red[2][c] + red[3][c]);
    }
  }
}

// Adds the chunks' partial rows: 64 columns per workgroup of sixteen waves, wave w takes chunks w, w + 16, ...,
// eight rows at a time (eight independent loads in flight per lane; a row past the last chunk is not loaded and
// counts as zero), and the waves meet in LDS: up to 128 chunks cost one round of loads.  The order of the
// additions is fixed.
constexpr int kFinishWaves = 16;
template <typename T>
__global__ __launch_bounds__(64 * kFinishWaves) void bias_gradient_finish_kernel(const float* partial, int chunks, int N,
                                                                                 typename T::storage* dbias, long long stride) {
  __shared__ float red[kFinishWaves][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = blockIdx.x * 64 + lane;
  float s[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) s[i] = 0.0f;
  if (n < N) {
    for (int c = wave; c < chunks; c += 8 * kFinishWaves) {
      float v[8];
#pragma unroll
      for (int i = 0; i < 8; ++i)
        v[i] = c + kFinishWaves * i < chunks ? partial[(long long)(c + kFinishWaves * i) * N + n] : 0.0f;
#pragma unroll
      for (int i = 0; i < 8; ++i) s[i] += v[i];
    }
  }
  red[wave][lane] = ((s[0] + s[1]) + (s[2] + s[3])) + ((s[4] + s[5]) + (s[6] + s[7]));
  __syncthreads();
  if (wave == 0 && n < N) {
    float t[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) t[i] = (red[4 * i][lane] + red[4 * i + 1][lane]) + (red[4 * i + 2][lane] + red[4 * i + 3][lane]);
    dbias[(long long)n * stride] = T::from_float((t[0] + t[1]) + (t[2] + t[3]));
  }
}

// Scratch of the entry point that allocates nothing (srtActivationBackwardBiasNoAlloc): the chunks'
// partial bias-gradient rows, [chunks][N] fp32.  One copy per device, held until the process ends;
// kScratchBytes is the entry point's size limit.  Host code never passes the array's name to a
// kernel: it asks the runtime for the device's address of it once per device and uses that pointer.
constexpr size_t kScratchBytes = 8u << 20;
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[kScratchBytes];

// Device `device`'s address of `scratch`, resolved once per device with that device current and cached.
// srtStreamCreate resolves it for its stream's device (prepare_backward_scratch), so a call on a stream this
// library created finds it cached; for a stream made elsewhere the first call per device resolves it here.
std::atomic<void*> scratch_address[64];

float* scratch_of_device(int device, srtStatus* status) {
  if (device < 0 || device >= 64) {
    *status = srtErrorNoDevice;
    return nullptr;
  }
  void* ptr = scratch_address[device].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    int current = -1;
    hipError_t e = hipGetDevice(&current);
    const bool other = e == hipSuccess && current != device;
    if (other) e = hipSetDevice(device);
    if (e == hipSuccess) e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (other) (void)hipSetDevice(current);
    if (e != hipSuccess || ptr == nullptr) {
      (void)hipGetLastError();
      *status = e == hipSuccess ? srtErrorUnknown : from_hip(e);
      return nullptr;
    }
    scratch_address[device].store(ptr, std::memory_order_release);
  }
  *status = srtSuccess;
  return static_cast<float*>(ptr);
}

// The array of the device `stream` belongs to (the null stream: the current device).
float* scratch_of_stream(hipStream_t stream, srtStatus* status) {
  int device = -1;
  const hipError_t e = stream ? hipStreamGetDevice(stream, &device) : hipGetDevice(&device);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    *status = from_hip(e);
    return nullptr;
  }
  return scratch_of_device(device, status);
}

// fixed_workspace: false -- the partial rows come from the library's stream-ordered allocator;
// true -- from the device's static scratch array (nothing is allocated or freed), and a problem
// whose partial rows exceed it is refused.
template <typename T>
srtStatus run(BackwardProblem p, void* dbias, long long dbias_stride, hipStream_t stream, bool fixed_workspace) {
  constexpr int VEC = 16 / sizeof(typename T::storage);
  const size_t es = sizeof(typename T::storage);
  auto vec_ok = [&](const void* ptr, long long sm, long long sn) {
    return sn == 1 && sm % VEC == 0 && (uintptr_t)ptr % (VEC * es) == 0;
  };
  const bool vec = p.N % VEC == 0 && vec_ok(p.y, p.sym, p.syn) && vec_ok(p.dy, p.sdm, p.sdn) && vec_ok(p.dx, p.sxm, p.sxn);
  const int V = vec ? VEC : 1;
  const int strips = (p.N + 64 * V - 1) / (64 * V);
  // enough workgroups to keep every memory channel busy, but at least 16 rows per chunk
  // (1024 to 6144 workgroups and one, two or four rows per trip all measure the same on 4096 x 11008; fewer chunks
  // are fewer partial rows for the second kernel)
  int chunks = (2048 + strips - 1) / strips;
  const int max_chunks = (p.M + 15) / 16;
  if (chunks > max_chunks) chunks = max_chunks;
  if (chunks > 65535) chunks = 65535;
  // the chunks' partial rows fit the fixed workspace of the entry point that does not allocate whenever
  // a single row does (both entry points cut the rows the same way, so their sums agree bit for bit)
  const long long fit = (long long)(kScratchBytes / sizeof(float)) / p.N;
  if (chunks > fit) chunks = (int)fit;
  if (chunks < 1) chunks = 1;
  p.rows_per_chunk = (p.M + chunks - 1) / chunks;
  chunks = (p.M + p.rows_per_chunk - 1) / p.rows_per_chunk;

  void* workspace = nullptr;
  if (dbias && fixed_workspace) {
    if ((size_t)chunks * p.N * sizeof(float) > kScratchBytes) return srtErrorInvalidValue;
    srtStatus s;
    workspace = scratch_of_stream(stream, &s);
    if (!workspace) return s;
    // every entry the second kernel reads is written by the first (all chunks, all N columns), so the
    // previous call's contents need no clearing
  } else if (dbias) {
    srtStatus s = srtDeviceAllocate(&workspace, (size_t)chunks * p.N * sizeof(float), reinterpret_cast<srtStream>(stream));
    if (s != srtSuccess) return s;
  }
  p.partial = (float*)workspace;
  const dim3 grid(strips, chunks);
  if (vec) hipLaunchKernelGGL((activation_backward_kernel<T, VEC, 2>), grid, dim3(256), 0, stream, p);
  else hipLaunchKernelGGL((activation_backward_kernel<T, 1, 2>), grid, dim3(256), 0, stream, p);
  hipError_t e = launch_status(stream);
  if (e == hipSuccess && dbias) {
    hipLaunchKernelGGL((bias_gradient_finish_kernel<T>), dim3((p.N + 63) / 64), dim3(64 * kFinishWaves), 0, stream,
                       (const float*)workspace, chunks, p.N, (typename T::storage*)dbias, dbias_stride);
    e = launch_status(stream);
  }
  // stream-ordered: the block becomes reusable for other streams only after the work queued so
  // far on `stream` has finished
  if (workspace && !fixed_workspace) (void)srtDeviceFree(workspace);
  return from_hip(e);
}

}  // namespace

// Set-up hook of the runtime (srtStreamCreate): resolves the current device's scratch address ahead of the first
// srtActivationBackwardBiasNoAlloc, whose calls then touch no runtime state beyond their launches.
void prepare_backward_scratch() {
  int device = -1;
  srtStatus ignored;
  if (hipGetDevice(&device) == hipSuccess) (void)scratch_of_device(device, &ignored);
  else (void)hipGetLastError();
}
}  // namespace srt

static srtStatus activation_backward_bias(const void* y, const srtTensorDescriptor* yDesc, const void* dy,
                                          const srtTensorDescriptor* dyDesc, srtActivation activation,
                                          double coef, void* dx, const srtTensorDescriptor* dxDesc,
                                          void* dbias, const srtTensorDescriptor* dbiasDesc,
                                          srtStream stream, bool fixed_workspace) {
  auto ok = [](const srtTensorDescriptor* d) { return d && d->shape && d->strides; };
  if (!ok(yDesc) || !ok(dyDesc) || !ok(dxDesc)) return srtErrorInvalidValue;
  if (dxDesc->rank != 2) return srtErrorNotSupported;
  if (yDesc->rank != 2 || dyDesc->rank != 2) return srtErrorInvalidValue;
  const srtDataType t = dxDesc->type;
  if (t != srtReal32F && t != srtReal16F && t != srtReal16BF) return srtErrorNotSupported;
  if (yDesc->type != t || dyDesc->type != t) return srtErrorNotSupported;
  if ((unsigned)activation > (unsigned)srtActivationIdentity) return srtErrorInvalidValue;
  const size_t M = dxDesc->shape[0], N = dxDesc->shape[1];
  if (yDesc->shape[0] != M || yDesc->shape[1] != N || dyDesc->shape[0] != M || dyDesc->shape[1] != N)
    return srtErrorInvalidValue;
  long long dbias_stride = 0;
  if (dbias) {
    if (!ok(dbiasDesc)) return srtErrorInvalidValue;
    if (dbiasDesc->type != t) return srtErrorNotSupported;
    if (dbiasDesc->rank != 1 || dbiasDesc->shape[0] != N) return srtErrorInvalidValue;
    dbias_stride = (long long)dbiasDesc->strides[0];
  }
  if (M > 0x7fffffffu || N > 0x7fffffffu) return srtErrorNotSupported;
  if (N == 0) return srtSuccess;
  if (M == 0) {
    // an empty sum: the bias gradient is zero
    if (dbias) {
      const uint32_t zero = 0;
      if (dbias_stride != 1) return srtErrorNotSupported;
      return srtFillFlat(t, dbias, &zero, N, stream);
    }
    return srtSuccess;
  }
  if (!y || !dy || !dx) return srtErrorInvalidValue;
  srt::BackwardProblem p{};
  p.M = (int)M; p.N = (int)N;
  p.y = y; p.dy = dy; p.dx = dx;
  p.sym = (long long)yDesc->strides[0]; p.syn = (long long)yDesc->strides[1];
  p.sdm = (long long)dyDesc->strides[0]; p.sdn = (long long)dyDesc->strides[1];
  p.sxm = (long long)dxDesc->strides[0]; p.sxn = (long long)dxDesc->strides[1];
  p.activation = (int)activation;
  p.coef = (float)coef;
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  switch (t) {
    case srtReal32F: return srt::run<srt::F32>(p, dbias, dbias_stride, hs, fixed_workspace);
    case srtReal16F: return srt::run<srt::F16>(p, dbias, dbias_stride, hs, fixed_workspace);
    default: return srt::run<srt::BF16>(p, dbias, dbias_stride, hs, fixed_workspace);
  }
}

extern "C" srtStatus srtActivationBackwardBias(const void* y, const srtTensorDescriptor* yDesc, const void* dy,
                                               const srtTensorDescriptor* dyDesc, srtActivation activation,
                                               double coef, void* dx, const srtTensorDescriptor* dxDesc,
                                               void* dbias, const srtTensorDescriptor* dbiasDesc,
                                               srtStream stream) {
  return activation_backward_bias(y, yDesc, dy, dyDesc, activation, coef, dx, dxDesc, dbias, dbiasDesc, stream, false);
}

extern "C" srtStatus srtActivationBackwardBiasNoAlloc(const void* y, const srtTensorDescriptor* yDesc, const void* dy,
                                                      const srtTensorDescriptor* dyDesc, srtActivation activation,
                                                      double coef, void* dx, const srtTensorDescriptor* dxDesc,
                                                      void* dbias, const srtTensorDescriptor* dbiasDesc,
                                                      srtStream stream) {
  return activation_backward_bias(y, yDesc, dy, dyDesc, activation, coef, dx, dxDesc, dbias, dbiasDesc, stream, true);
}
