// Generic strided matmul: any element type of the path, any strides (views, column-major,
// non-unit inner strides), any extents.  LDS-tiled 64x64x16, fp32 FMA accumulation.
// This is the layout-complete kernel; the MFMA and skinny kernels take the aligned
// fast cases and everything else lands here.
#include "gemm_common.h"

namespace srt {

namespace {

constexpr int GT = 64;   // tile edge (M and N)
constexpr int GK = 16;   // k depth per stage

template <typename T>
__global__ __launch_bounds__(256) void gemm_generic_kernel(GemmProblem p) {
  using S = typename T::storage;
  __shared__ float As[GK][GT + 4];
  __shared__ float Bs[GK][GT + 4];

  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
  const int bz = blockIdx.z;
  const S* A = (const S*)p.A + (long long)bz * p.sab;
  const S* B = (const S*)p.B + (long long)bz * p.sbb;
  S* C = (S*)p.C + (long long)bz * p.scb;

  // pick the thread -> element mapping that walks the unit stride first
  const bool a_k_fast = (p.sak == 1);
  const bool b_n_fast = (p.sbn == 1);

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;

  for (int k0 = 0; k0 < p.K; k0 += GK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int idx = tid + i * 256;
      int mm, kk;
      if (a_k_fast) { kk = idx & (GK - 1); mm = idx >> 4; } else { mm = idx & (GT - 1); kk = idx >> 6; }
      int m = m0 + mm, k = k0 + kk;
      float v = 0.0f;
      if (m < p.M && k < p.K) v = T::to_float(A[(long long)m * p.sam + (long long)k * p.sak]);
      As[kk][mm] = v;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int idx = tid + i * 256;
      int nn, kk;
      if (b_n_fast) { nn = idx & (GT - 1); kk = idx >> 6; } else { kk = idx & (GK - 1); nn = idx >> 4; }
      int n = n0 + nn, k = k0 + kk;
      float v = 0.0f;
      if (n < p.N && k < p.K) v = T::to_float(B[(long long)k * p.sbk + (long long)n * p.sbn]);
      Bs[kk][nn] = v;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Bs[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }

  Epilogue<T> ep(p);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int m = m0 + ty * 4 + i;
    if (m >= p.M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int n = n0 + tx * 4 + j;
      if (n >= p.N) continue;
      C[(long long)m * p.scm + (long long)n * p.scn] = ep.finish(acc[i][j], ep.bias_at(m, n));
    }
  }
}

}  // namespace

bool generic_supported(const GemmProblem& p) {
  if (p.dtype != srtReal32F && p.dtype != srtReal16F && p.dtype != srtReal16BF) return false;
  // grid limits: y and z dimensions hold at most 65535 blocks
  if ((p.M + GT - 1) / GT > 65535 || p.batch > 65535) return false;
  return true;
}

hipError_t launch_generic(const GemmProblem& p, hipStream_t stream) {
  dim3 grid((p.N + GT - 1) / GT, (p.M + GT - 1) / GT, p.batch);
  dim3 block(256);
  switch (p.dtype) {
    case srtReal32F: hipLaunchKernelGGL(gemm_generic_kernel<F32>, grid, block, 0, stream, p); break;
    case srtReal16F: hipLaunchKernelGGL(gemm_generic_kernel<F16>, grid, block, 0, stream, p); break;
    case srtReal16BF: hipLaunchKernelGGL(gemm_generic_kernel<BF16>, grid, block, 0, stream, p); break;
    default: return hipErrorNotSupported;
  }
  return launch_status(stream);
}

}  // namespace srt
