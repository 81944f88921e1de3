// srtMatmul / srtMatmulBiasActivation: descriptor validation, folding of transposes, orders
// and views into one strided problem, and kernel-family selection.
#include <cstdio>
#include <cstring>

#include "gemm_common.h"
#include "status.h"

namespace {

using srt::GemmProblem;

bool supported_type(srtDataType t) { return t == srtReal32F || t == srtReal16F || t == srtReal16BF; }

// Builds the normalized problem.  Returns srtSuccess, srtErrorNotSupported (caller falls
// back to the CPU) or srtErrorInvalidValue.  *empty is set when an extent is zero.
srtStatus build_problem(const void* a, const srtTensorDescriptor* ad, int tA,
                        const void* b, const srtTensorDescriptor* bd, int tB,
                        const void* bias, const srtTensorDescriptor* biasd, int activation, double coef,
                        void* out, const srtTensorDescriptor* od, GemmProblem* p, bool* empty) {
  *empty = false;
  if (!ad || !bd || !od) return srtErrorInvalidValue;
  if (!ad->shape || !ad->strides || !bd->shape || !bd->strides || !od->shape || !od->strides)
    return srtErrorInvalidValue;
  const uint32_t rank = od->rank;
  if (rank != 2 && rank != 3) return srtErrorNotSupported;
  if (ad->rank != rank || bd->rank != rank) return srtErrorInvalidValue;
  if (!supported_type(od->type)) return srtErrorNotSupported;
  if (ad->type != od->type || bd->type != od->type) return srtErrorNotSupported;
  auto order_ok = [](srtOrder o) { return o == srtOrderRow || o == srtOrderCol; };
  if (!order_ok(ad->order) || !order_ok(bd->order) || !order_ok(od->order)) return srtErrorNotSupported;
  if ((unsigned)activation > (unsigned)srtActivationIdentity) return srtErrorInvalidValue;

  const uint32_t r = rank - 2;
  size_t am = ad->shape[r], ak = ad->shape[r + 1], sam = ad->strides[r], sak = ad->strides[r + 1];
  if (tA) { size_t t = am; am = ak; ak = t; t = sam; sam = sak; sak = t; }
  size_t bk = bd->shape[r], bn = bd->shape[r + 1], sbk = bd->strides[r], sbn = bd->strides[r + 1];
  if (tB) { size_t t = bk; bk = bn; bn = t; t = sbk; sbk = sbn; sbn = t; }
  const size_t M = od->shape[r], N = od->shape[r + 1];
  if (am != M || bn != N || ak != bk) return srtErrorInvalidValue;
  size_t batch = 1;
  if (rank == 3) {
    batch = od->shape[0];
    if (ad->shape[0] != batch || bd->shape[0] != batch) return srtErrorInvalidValue;
  }
  const size_t lim = 0x7fffffffu;
  if (M > lim || N > lim || ak > lim || batch > lim) return srtErrorNotSupported;

  p->dtype = od->type;
  p->M = (int)M; p->N = (int)N; p->K = (int)ak; p->batch = (int)batch;
  p->A = a; p->B = b; p->C = out;
  p->sam = (long long)sam; p->sak = (long long)sak; p->sab = rank == 3 ? (long long)ad->strides[0] : 0;
  p->sbk = (long long)sbk; p->sbn = (long long)sbn; p->sbb = rank == 3 ? (long long)bd->strides[0] : 0;
  p->scm = (long long)od->strides[r]; p->scn = (long long)od->strides[r + 1];
  p->scb = rank == 3 ? (long long)od->strides[0] : 0;
  p->bias = nullptr; p->sbias = 0; p->bias_per_row = 0;
  p->activation = activation; p->coef = (float)coef;
  if (bias) {
    if (!biasd || !biasd->shape || !biasd->strides) return srtErrorInvalidValue;
    if (biasd->type != od->type) return srtErrorNotSupported;
    if (biasd->rank != 1 || biasd->shape[0] != N) return srtErrorInvalidValue;
    p->bias = bias; p->sbias = (long long)biasd->strides[0];
  }
  if (M == 0 || N == 0 || batch == 0) { *empty = true; return srtSuccess; }
  if (!a || !b || !out) return srtErrorInvalidValue;

  // Column-major (or otherwise M-contiguous) result: compute C^T = op(B)^T . op(A)^T so the
  // kernels always write rows with the smaller stride innermost.
  if (p->scn != 1 && p->scm == 1) {
    GemmProblem q = *p;
    q.M = p->N; q.N = p->M;
    q.A = p->B; q.sam = p->sbn; q.sak = p->sbk; q.sab = p->sbb;
    q.B = p->A; q.sbk = p->sak; q.sbn = p->sam; q.sbb = p->sab;
    q.scm = p->scn; q.scn = p->scm;
    q.bias_per_row = 1;
    *p = q;
  }
  return srtSuccess;
}

enum Family { kGeneric, kMfma, kSkinny, kF32Mfma };

Family select(const GemmProblem& p, int* config) {
  *config = 0;
  if (srt::skinny_supported(p)) return kSkinny;
  int c = srt::mfma_select(p);
  if (c) { *config = c; return kMfma; }
  if (srt::f32_mfma_supported(p)) return kF32Mfma;
  return kGeneric;
}

srtStatus run(const GemmProblem& p, hipStream_t stream) {
  int config = 0;
  hipError_t e;
  switch (select(p, &config)) {
    case kSkinny: e = srt::launch_skinny(p, stream); break;
    case kMfma: e = srt::launch_mfma(p, config, stream); break;
    case kF32Mfma: e = srt::launch_f32_mfma(p, stream); break;
    default:
      if (!srt::generic_supported(p)) return srtErrorNotSupported;
      e = srt::launch_generic(p, stream);
  }
  return srt::from_hip(e);
}

}  // namespace

extern "C" {

srtStatus srtMatmulBiasActivation(const void* a, const srtTensorDescriptor* aDesc, int32_t transposeA,
                                  const void* b, const srtTensorDescriptor* bDesc, int32_t transposeB,
                                  const void* bias, const srtTensorDescriptor* biasDesc,
                                  srtActivation activation, double coef,
                                  void* out, const srtTensorDescriptor* oDesc, srtStream stream) {
  GemmProblem p;
  bool empty = false;
  srtStatus s = build_problem(a, aDesc, transposeA, b, bDesc, transposeB, bias, biasDesc, (int)activation, coef,
                              out, oDesc, &p, &empty);
  if (s != srtSuccess || empty) return s;
  return run(p, reinterpret_cast<hipStream_t>(stream));
}

srtStatus srtMatmul(const void* a, const srtTensorDescriptor* aDesc, int32_t transposeA,
                    const void* b, const srtTensorDescriptor* bDesc, int32_t transposeB,
                    void* out, const srtTensorDescriptor* oDesc, srtStream stream) {
  return srtMatmulBiasActivation(a, aDesc, transposeA, b, bDesc, transposeB, nullptr, nullptr,
                                 srtActivationIdentity, 0.0, out, oDesc, stream);
}

srtStatus srtMatmulQueryKernel(const srtTensorDescriptor* aDesc, int32_t transposeA,
                               const srtTensorDescriptor* bDesc, int32_t transposeB,
                               const srtTensorDescriptor* oDesc, const void* a, const void* b,
                               const void* out, char* name, size_t nameCapacity) {
  if (!name || nameCapacity == 0) return srtErrorInvalidValue;
  name[0] = 0;
  GemmProblem p;
  bool empty = false;
  srtStatus s = build_problem(a, aDesc, transposeA, b, bDesc, transposeB, nullptr, nullptr,
                              srtActivationIdentity, 0.0, const_cast<void*>(out), oDesc, &p, &empty);
  if (s != srtSuccess) return s;
  const char* n = "generic";
  if (empty) n = "empty";
  else {
    int config = 0;
    switch (select(p, &config)) {
      case kSkinny: n = "skinny"; break;
      case kMfma: n = srt::mfma_name(config); break;
      case kF32Mfma: n = "f32_mfma"; break;
      default: n = "generic";
    }
  }
  std::snprintf(name, nameCapacity, "%s", n);
  return srtSuccess;
}

}  // extern "C"
