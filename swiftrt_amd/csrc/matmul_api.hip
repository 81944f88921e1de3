// srtMatmul / srtMatmulBiasActivation: descriptor validation, folding of transposes, orders
// and views into one strided problem, and kernel-family selection.
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <tuple>

#include "gemm_common.h"
#include "status.h"
#include "views.h"

namespace {

using srt::GemmProblem;

bool supported_type(srtDataType t) { return t == srtReal32F || t == srtReal16F || t == srtReal16BF; }

// Builds the normalized problem.  Returns srtSuccess, srtErrorNotSupported (caller falls
// back to the CPU) or srtErrorInvalidValue.  *empty is set when an extent is zero.
srtStatus build_problem(const void* a, const srtTensorDescriptor* ad, int tA,
                        const void* b, const srtTensorDescriptor* bd, int tB,
                        const void* bias, const srtTensorDescriptor* biasd, int activation, double coef,
                        void* out, const srtTensorDescriptor* od, GemmProblem* p, bool* empty,
                        bool check_alias = true) {
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
  p->activation = activation; p->coef = (float)coef; p->tile_n = 0;
  if (bias) {
    if (!biasd || !biasd->shape || !biasd->strides) return srtErrorInvalidValue;
    if (biasd->type != od->type) return srtErrorNotSupported;
    if (biasd->rank != 1 || biasd->shape[0] != N) return srtErrorInvalidValue;
    p->bias = bias; p->sbias = (long long)biasd->strides[0];
  }
  if (M == 0 || N == 0 || batch == 0) { *empty = true; return srtSuccess; }
  if (!a || !b || !out) return srtErrorInvalidValue;

  // The kernels read operand tiles while other workgroups already store results, so the result must share no
  // element with an input (the Swift side always hands in a freshly allocated dense result,
  // operators/Matmul.swift:38-39).  Storage spans that do not overlap settle it.  Views whose spans do overlap
  // are accepted when a common pitch proves them apart (column slices of one wide buffer, interleaved
  // batches: see views_disjoint); a result that provably shares an element with an input (the same first element, or overlapping row blocks
  // of one pitch) is an error; anything else
  // is answered "not supported", so that the caller's fallback runs instead of a wrong guess either way.
  if (check_alias) {   // (the kernel query takes placeholder pointers and launches nothing)
    const size_t es = od->type == srtReal32F ? 4 : 2;
    const srt::StridedView vo = srt::make_view(out, es, p->M, p->scm, p->N, p->scn, p->batch, p->scb);
    auto verdict = [&](const srt::StridedView& v) {
      if (!srt::spans_overlap(vo, v)) return srtSuccess;
      if (srt::views_alias(vo, v)) return srtErrorInvalidValue;
      return srt::views_disjoint(vo, v) ? srtSuccess : srtErrorNotSupported;
    };
    if (p->K > 0) {
      if (srtStatus s = verdict(srt::make_view(a, es, p->M, p->sam, p->K, p->sak, p->batch, p->sab)); s != srtSuccess) return s;
      if (srtStatus s = verdict(srt::make_view(b, es, p->K, p->sbk, p->N, p->sbn, p->batch, p->sbb)); s != srtSuccess) return s;
    }
    if (bias) {
      if (srtStatus s = verdict(srt::make_view(bias, es, p->N, p->sbias, 1, 0, 1, 0)); s != srtSuccess) return s;
    }
  }

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

// ---- plans ------------------------------------------------------------------------------------
// A plan names the kernel that runs a problem.  The heuristic picks one per call; srtMatmulTune
// measures every plan the problem qualifies for and records the fastest in a process-wide cache
// keyed by the problem's shape, layout class and epilogue, which later calls consult first
// (the role of ExecutionPlanCache / ExecutionPlanner, platform/common/ExecutionPlanner.swift:20-29,
// and of the empty CudaMatmul2.tune, platform/cuda/functions/CudaMatmul.swift:112-120).
enum Plan { kPlanGeneric, kPlanSkinny, kPlanRing256, kPlanMfma128, kPlanMfma64, kPlanF32Tile64, kPlanF32SplitK,
            kPlanKc64, kPlanM16, kPlanSplitK, kPlanM16H, kPlanAny128, kPlanAny64, kPlanM16D, kPlanM16DTail, kPlanM16DSplit, kPlanM16DH, kPlanM16DN, kPlanM16Q, kPlanF32Parts, kPlanF32Ring, kPlanF32Ring64x128, kPlanF32Ring64, kPlanCount };

const char* const kPlanNames[kPlanCount] = {"generic", "skinny", "mfma_256x256", "mfma_128x128", "mfma_64x64",
                                            "f32_mfma_64x64", "f32_mfma_splitk", "mfma_256x256_k64",
                                            "mfma_256x256_m16", "mfma_256x256_splitk", "mfma_128x256_m16",
                                            "mfma_128x128_any", "mfma_64x64_any", "mfma_256x256_m16_k64",
                                            "mfma_256x256_m16_k64_tail", "mfma_256x256_m16_k64_split",
                                            "mfma_128x256_m16_k64", "mfma_256x128_m16_k64", "mfma_128x128_m16_k128", "f32_mfma_128x128_parts", "f32_mfma_128x128_ring", "f32_mfma_64x128_ring", "f32_mfma_64x64_ring"};

bool plan_supported(const GemmProblem& p, Plan plan) {
  switch (plan) {
    case kPlanSkinny: return srt::skinny_supported(p);
    case kPlanRing256: return srt::mfma_config(p, 1) != 0;
    case kPlanMfma128: return srt::mfma_config(p, 2) != 0;
    case kPlanMfma64: return srt::mfma_config(p, 3) != 0;
    case kPlanKc64: return srt::mfma_config(p, 4) != 0;
    case kPlanM16: return srt::mfma_config(p, 5) != 0;
    case kPlanSplitK: return srt::mfma_splitk_parts(p) >= 2;
    case kPlanM16H: return srt::mfma_config(p, 6) != 0;
    case kPlanAny128: return srt::mfma_config(p, 7) != 0;
    case kPlanAny64: return srt::mfma_config(p, 8) != 0;
    case kPlanM16D: return srt::mfma_config(p, 9) != 0;
    case kPlanM16DTail: return srt::mfma_config(p, 10) != 0;
    case kPlanM16DSplit: return srt::mfma_config(p, 11) != 0;
    case kPlanM16DH: return srt::mfma_config(p, 12) != 0;
    case kPlanM16DN: return srt::mfma_config(p, 13) != 0;
    case kPlanM16Q: return srt::mfma_config(p, 14) != 0;
    case kPlanF32Parts: return srt::f32_mfma_supported(p) && srt::f32_tile_parts(p) >= 2;
    case kPlanF32Ring:
    case kPlanF32Ring64x128:
    case kPlanF32Ring64: return srt::f32_ring_fits(p);
    case kPlanF32Tile64: return srt::f32_mfma_supported(p) && (p.M + 63) / 64 <= 65535;
    case kPlanF32SplitK: return srt::f32_mfma_supported(p);
    default: return srt::generic_supported(p);
  }
}

Plan heuristic_plan(const GemmProblem& p) {
  // one round of 128 x 128 tiles holds the problem (64 rows or more) and its k loop is not worth cutting
  if (srt::mfma_prefers_quarter(p)) return kPlanM16Q;
  if (srt::skinny_supported(p) && srt::skinny_preferred(p)) return kPlanSkinny;
  // Up to 64 rows against a long k loop, one round of the streaming kernel's workgroups: when split-K cannot cut the k
  // loop, or only in two (K / 4 not a whole number of stages; a batch has no split-K pass at all), the streaming kernel beats
  // tiles that leave most of the device idle (24 x 96 x 10320: 32 us against 121 in half tiles; 64 x 144 x 8400 x . W^T: 26
  // against 61 in 64 x 64 tiles; 8 x 1288 x 10432: 44 against 58 in two parts).  With up to 32 rows that is decided ahead
  // of tail sharing, whose tiles would be nearly all padding (28 x 8 x 88 x 7680: 32 us against 59).
  const bool streams = p.dtype != srtReal32F && p.K >= 2048 && srt::skinny_supported(p) && (long long)((p.N + 63) / 64) * p.batch <= 256;
  const bool few_parts = srt::mfma_splitk_parts(p) <= 2;
  if (streams && few_parts && p.M <= 32) return kPlanSkinny;
  // tiles left over after the whole rounds and a long k loop: cut along k for the idle compute units
  if (srt::mfma_prefers_tail(p)) return kPlanM16DTail;
  // (The split form -- whole rounds of whole tiles, then one round of 192-wide ones -- is never the heuristic's choice:
  // on this power-limited device the compute units that idle through a ragged last round lend their power to the busy
  // ones, and the form measures the same as whole tiles or worse.  4096 x 11008 x 4096, 2.69 rounds, same run: 249-257 us
  // whole, 254-258 split; 2048 x 13000 x 4096, 1.59 rounds: 158-162 against 168-170.  srtMatmulTune still times it.)
  if (streams && few_parts) return kPlanSkinny;
  // few 256 x 256 tiles and a long k loop: K split over the idle compute units
  if (srt::mfma_prefers_splitk(p)) return kPlanSplitK;
  if (streams) return kPlanSkinny;
  const int c = srt::mfma_select(p);
  if (c) {
    switch (c >> 2) {
      case 1: return kPlanRing256;
      case 2: return kPlanMfma128;
      case 4: return kPlanKc64;
      case 5: return kPlanM16;
      case 6: return kPlanM16H;
      case 7: return kPlanAny128;
      case 8: return kPlanAny64;
      case 9: return kPlanM16D;
      case 10: return kPlanM16DTail;
      case 12: return kPlanM16DH;
      case 13: return kPlanM16DN;
      case 14: return kPlanM16Q;
      default: return kPlanMfma64;
    }
  }
  if (srt::f32_mfma_supported(p)) {
    // what the ring kernel reads: the fastest of its three tile shapes, the k range in parts and the 32 x 32 kernel,
    // by their time estimates
    if (srt::f32_ring_fits(p)) {
      switch (srt::f32_ring_choice(p)) {
        case 0: return kPlanF32Ring;
        case 1: return kPlanF32Ring64x128;
        case 2: return kPlanF32Ring64;
        case 3: return kPlanF32Parts;
        default: return kPlanF32SplitK;
      }
    }
    // launch-sized problems and up to 64 rows: 32 x 32 tiles whose four waves split K
    if (srt::f32_mfma_prefers_splitk(p)) return kPlanF32SplitK;
    // a single matrix of too few 128 x 128 tiles for the device: its k range in parts on those tiles
    if (srt::f32_tile_parts(p) >= 2) return kPlanF32Parts;
    return kPlanF32Tile64;
  }
  return kPlanGeneric;
}

hipError_t launch_plan(const GemmProblem& p, Plan plan, hipStream_t stream) {
  switch (plan) {
    case kPlanSkinny: return srt::launch_skinny(p, stream);
    case kPlanRing256: return srt::launch_mfma(p, srt::mfma_config(p, 1), stream);
    case kPlanMfma128: return srt::launch_mfma(p, srt::mfma_config(p, 2), stream);
    case kPlanMfma64: return srt::launch_mfma(p, srt::mfma_config(p, 3), stream);
    case kPlanKc64: return srt::launch_mfma(p, srt::mfma_config(p, 4), stream);
    case kPlanM16: return srt::launch_mfma(p, srt::mfma_config(p, 5), stream);
    case kPlanSplitK: return srt::launch_mfma_splitk(p, stream);
    case kPlanM16H: return srt::launch_mfma(p, srt::mfma_config(p, 6), stream);
    case kPlanAny128: return srt::launch_mfma(p, srt::mfma_config(p, 7), stream);
    case kPlanAny64: return srt::launch_mfma(p, srt::mfma_config(p, 8), stream);
    case kPlanM16D: return srt::launch_mfma(p, srt::mfma_config(p, 9), stream);
    case kPlanM16DTail: return srt::launch_mfma(p, srt::mfma_config(p, 10), stream);
    case kPlanM16DSplit: return srt::launch_mfma(p, srt::mfma_config(p, 11), stream);
    case kPlanM16DH: return srt::launch_mfma(p, srt::mfma_config(p, 12), stream);
    case kPlanM16DN: return srt::launch_mfma(p, srt::mfma_config(p, 13), stream);
    case kPlanM16Q: return srt::launch_mfma(p, srt::mfma_config(p, 14), stream);
    case kPlanF32Parts: return srt::launch_f32_tile_parts(p, stream);
    case kPlanF32Ring: return srt::launch_f32_ring(p, stream, 0);
    case kPlanF32Ring64x128: return srt::launch_f32_ring(p, stream, 1);
    case kPlanF32Ring64: return srt::launch_f32_ring(p, stream, 2);
    case kPlanF32Tile64: return srt::launch_f32_mfma_variant(p, false, stream);
    case kPlanF32SplitK: return srt::launch_f32_mfma_variant(p, true, stream);
    default: return srt::launch_generic(p, stream);
  }
}

struct PlanKey {
  int dtype, M, N, K, batch, layout, epilogue;
  bool operator<(const PlanKey& o) const {
    return std::tie(dtype, M, N, K, batch, layout, epilogue) <
           std::tie(o.dtype, o.M, o.N, o.K, o.batch, o.layout, o.epilogue);
  }
};

// Layout class: which dimension of each operand is contiguous (bits 0-1: A along k / m, bits 2-3:
// B along k / n), whether the batch strides are dense, and whether rows keep 16-byte alignment.
PlanKey key_of(const GemmProblem& p) {
  int layout = 0;
  if (p.sak == 1) layout |= 1;
  if (p.sam == 1) layout |= 2;
  if (p.sbk == 1) layout |= 4;
  if (p.sbn == 1) layout |= 8;
  if (p.scn == 1) layout |= 16;
  if (p.bias_per_row) layout |= 32;
  const long long lda = p.sak == 1 ? p.sam : p.sak, ldb = p.sbk == 1 ? p.sbn : p.sbk;
  if (lda % 8 == 0 && ldb % 8 == 0 && p.scm % 8 == 0) layout |= 64;
  const int epilogue = (p.bias ? 1 : 0) | (p.activation << 1);
  return PlanKey{p.dtype, p.M, p.N, p.K, p.batch, layout, epilogue};
}

class PlanCache {
 public:
  bool find(const PlanKey& k, Plan* plan) {
    std::lock_guard<std::mutex> lock(mu_);
    auto it = plans_.find(k);
    if (it == plans_.end()) return false;
    *plan = it->second;
    return true;
  }
  void put(const PlanKey& k, Plan plan) {
    std::lock_guard<std::mutex> lock(mu_);
    plans_[k] = plan;
  }
  void clear() {
    std::lock_guard<std::mutex> lock(mu_);
    plans_.clear();
  }
  size_t size() {
    std::lock_guard<std::mutex> lock(mu_);
    return plans_.size();
  }
  // One plan per line: dtype M N K batch layout epilogue plan-name
  srtStatus save(const char* path) {
    std::lock_guard<std::mutex> lock(mu_);
    FILE* f = std::fopen(path, "w");
    if (!f) return srtErrorInvalidValue;
    std::fprintf(f, "# SwiftRTHip matmul plans v1: dtype M N K batch layout epilogue plan\n");
    for (const auto& kv : plans_) {
      const PlanKey& k = kv.first;
      std::fprintf(f, "%d %d %d %d %d %d %d %s\n", k.dtype, k.M, k.N, k.K, k.batch, k.layout, k.epilogue,
                   kPlanNames[kv.second]);
    }
    return std::fclose(f) == 0 ? srtSuccess : srtErrorUnknown;
  }
  // All or nothing: a malformed line or an unknown plan name leaves the cache as it was.
  srtStatus load(const char* path) {
    FILE* f = std::fopen(path, "r");
    if (!f) return srtErrorInvalidValue;
    std::map<PlanKey, Plan> read;
    char line[256];
    bool ok = true;
    while (ok && std::fgets(line, sizeof(line), f)) {
      if (line[0] == '#' || line[0] == '\n') continue;
      PlanKey k;
      char name[64];
      if (std::sscanf(line, "%d %d %d %d %d %d %d %63s", &k.dtype, &k.M, &k.N, &k.K, &k.batch, &k.layout,
                      &k.epilogue, name) != 8) { ok = false; break; }
      int plan = -1;
      for (int i = 0; i < kPlanCount; ++i)
        if (std::strcmp(name, kPlanNames[i]) == 0) plan = i;
      if (plan < 0 || k.M < 0 || k.N < 0 || k.K < 0 || k.batch < 0) { ok = false; break; }
      read[k] = (Plan)plan;
    }
    std::fclose(f);
    if (!ok) return srtErrorInvalidValue;
    std::lock_guard<std::mutex> lock(mu_);
    for (const auto& kv : read) plans_[kv.first] = kv.second;
    return srtSuccess;
  }

 private:
  std::mutex mu_;
  std::map<PlanKey, Plan> plans_;
};

PlanCache& plan_cache() {
  static PlanCache* cache = new PlanCache();   // never destroyed: calls may race with process exit
  return *cache;
}

// The plan a call runs: the cached one when it still qualifies (alignment of this call's pointers
// is not part of the key), else the heuristic's.
Plan select(const GemmProblem& p) {
  Plan plan;
  if (plan_cache().size() != 0 && plan_cache().find(key_of(p), &plan) && plan_supported(p, plan)) return plan;
  return heuristic_plan(p);
}

// ---- operands beyond the 256 x 256 kernels' reach -------------------------------------------------
// The 256 x 256 kernels address every operand through one buffer descriptor and 32-bit byte
// offsets, so each operand tensor of a launch (all batches) must span less than 1 Gi elements.
// A device with hundreds of GB holds larger ones (262144 x 8192 activations, 64 batches of
// 8192 x 8192): rather than hand those to the 128 x 128 kernel at half the rate, the call is cut
// into pieces that are within reach -- halves of the batch, then of M, then of N, at multiples of
// the tile size -- and the pieces run back to back on the caller's stream.  A piece is an ordinary
// problem (its own pointers, the same strides) and goes through the same plan selection.  An
// operand whose k walk alone exceeds the reach (K x leading stride >= 1 Gi elements when k is not
// its contiguous dimension) cannot be helped this way and keeps the smaller tiles.
bool fits_256(const GemmProblem& p) { return srt::mfma_config(p, 1) != 0; }

bool split_for_reach(const GemmProblem& p, GemmProblem* lo, GemmProblem* hi) {
  if (p.dtype != srtReal16BF && p.dtype != srtReal16F) return false;
  if (fits_256(p)) return false;
  const long long tiles = (long long)((p.M + 255) / 256) * ((p.N + 255) / 256) * p.batch;
  if (tiles < 128) return false;   // the small tiles are the choice there anyway
  GemmProblem q = p;
  q.batch = 1; q.M = p.M < 256 ? p.M : 256; q.N = p.N < 256 ? p.N : 256;
  if (!fits_256(q)) return false;   // alignment, or a k walk out of reach: not a matter of extent
  auto at = [](const void* base, long long elements) {
    return static_cast<const void*>(static_cast<const char*>(base) + elements * 2);   // 16-bit elements
  };
  *lo = p; *hi = p;
  if (p.batch > 1) {
    const int h = p.batch / 2;
    lo->batch = h; hi->batch = p.batch - h;
    hi->A = at(p.A, h * p.sab); hi->B = at(p.B, h * p.sbb);
    hi->C = const_cast<void*>(at(p.C, h * p.scb));
    return true;
  }
  GemmProblem qm = p; qm.M = q.M;   // would whole columns of tiles fit?
  const bool by_m = p.M > 256 && (fits_256(qm) || p.N <= 256);
  if (by_m) {
    const int m0 = ((p.M / 2 + 255) / 256) * 256;
    lo->M = m0; hi->M = p.M - m0;
    hi->A = at(p.A, m0 * p.sam);
    hi->C = const_cast<void*>(at(p.C, m0 * p.scm));
    if (p.bias && p.bias_per_row) hi->bias = at(p.bias, m0 * p.sbias);
    return true;
  }
  if (p.N <= 256) return false;
  const int n0 = ((p.N / 2 + 255) / 256) * 256;
  lo->N = n0; hi->N = p.N - n0;
  hi->B = at(p.B, n0 * p.sbn);
  hi->C = const_cast<void*>(at(p.C, n0 * p.scn));
  if (p.bias && !p.bias_per_row) hi->bias = at(p.bias, n0 * p.sbias);
  return true;
}

bool has_cached_plan(const GemmProblem& p) {
  Plan plan;
  return plan_cache().size() != 0 && plan_cache().find(key_of(p), &plan) && plan_supported(p, plan);
}

srtStatus run(const GemmProblem& p, hipStream_t stream) {
  GemmProblem lo, hi;
  if (!has_cached_plan(p) && split_for_reach(p, &lo, &hi)) {
    const srtStatus s = run(lo, stream);
    return s != srtSuccess ? s : run(hi, stream);
  }
  const Plan plan = select(p);
  if (plan == kPlanGeneric && !srt::generic_supported(p)) return srtErrorNotSupported;
  hipError_t e = launch_plan(p, plan, stream);
  if ((plan == kPlanSplitK || plan == kPlanM16DTail) && e == hipErrorOutOfMemory) {
    // no room for the workspace (nothing was launched): the plan that needs none
    (void)hipGetLastError();
    const int c = plan == kPlanM16DTail ? srt::mfma_config(p, 9) : srt::mfma_select(p);
    e = c ? srt::launch_mfma(p, c, stream) : srt::launch_generic(p, stream);
  }
  if (plan == kPlanF32Parts && e == hipErrorOutOfMemory) {
    // likewise for the fp32 parts: the whole k range per tile, no workspace
    (void)hipGetLastError();
    e = srt::f32_ring_fits(p) ? srt::launch_f32_ring(p, stream, 0) : srt::launch_f32_mfma_variant(p, false, stream);
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
                              srtActivationIdentity, 0.0, const_cast<void*>(out), oDesc, &p, &empty, false);
  if (s != srtSuccess) return s;
  const char* n = "empty";
  if (!empty) {
    // a call that runs in pieces reports its first piece's kernel, marked "/pieces"
    GemmProblem piece = p, lo, hi;
    bool pieces = false;
    while (!has_cached_plan(piece) && split_for_reach(piece, &lo, &hi)) { piece = lo; pieces = true; }
    const Plan plan = select(piece);
    n = kPlanNames[plan];
    if (plan == kPlanF32Tile64 || plan == kPlanF32SplitK || plan == kPlanF32Parts || plan == kPlanF32Ring || plan == kPlanF32Ring64x128 || plan == kPlanF32Ring64) n = "f32_mfma";   // one family name for the fp32 tiles
    if (pieces) {
      std::snprintf(name, nameCapacity, "%s/pieces", n);
      return srtSuccess;
    }
  }
  std::snprintf(name, nameCapacity, "%s", n);
  return srtSuccess;
}

srtStatus srtMatmulTune(const void* a, const srtTensorDescriptor* aDesc, int32_t transposeA,
                        const void* b, const srtTensorDescriptor* bDesc, int32_t transposeB,
                        const void* bias, const srtTensorDescriptor* biasDesc,
                        srtActivation activation, double coef,
                        void* out, const srtTensorDescriptor* oDesc, srtStream stream,
                        char* chosen, size_t chosenCapacity) {
  if (chosen && chosenCapacity) chosen[0] = 0;
  GemmProblem p;
  bool empty = false;
  srtStatus s = build_problem(a, aDesc, transposeA, b, bDesc, transposeB, bias, biasDesc, (int)activation, coef,
                              out, oDesc, &p, &empty);
  if (s != srtSuccess || empty) return s;
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  {
    // a problem that runs in pieces has no single plan to record: its pieces keep the heuristic
    GemmProblem lo, hi;
    if (!has_cached_plan(p) && split_for_reach(p, &lo, &hi)) {
      if (chosen && chosenCapacity) std::snprintf(chosen, chosenCapacity, "pieces");
      return run(p, hs);
    }
  }
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess) return srtErrorUnknown;
  if (hipEventCreate(&e1) != hipSuccess) { (void)hipEventDestroy(e0); return srtErrorUnknown; }
  const Plan fallback = heuristic_plan(p);
  Plan best = fallback;
  float best_ms = -1.0f;
  hipError_t err = hipSuccess;
  for (int c = 0; c < kPlanCount && err == hipSuccess; ++c) {
    const Plan plan = (Plan)c;
    if (!plan_supported(p, plan)) continue;
    // the FMA kernel is orders of magnitude slower on large problems: skip it when a matrix-core plan exists
    if (plan == kPlanGeneric && fallback != kPlanGeneric && 2.0 * p.M * p.N * p.K * p.batch > 1e9) continue;
    const int warm = 2, reps = 8;
    for (int i = 0; i < warm && err == hipSuccess; ++i) err = launch_plan(p, plan, hs);
    if ((plan == kPlanSplitK || plan == kPlanM16DTail || plan == kPlanF32Parts) && err == hipErrorOutOfMemory) {
      // no room for this plan's workspace (nothing was launched): it is not a candidate, as in run()
      (void)hipGetLastError();
      err = hipSuccess;
      continue;
    }
    if (err == hipSuccess) err = hipEventRecord(e0, hs);
    for (int i = 0; i < reps && err == hipSuccess; ++i) err = launch_plan(p, plan, hs);
    if (err == hipSuccess) err = hipEventRecord(e1, hs);
    if (err == hipSuccess) err = hipEventSynchronize(e1);
    float ms = 0.0f;
    if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
    if (err == hipSuccess && (best_ms < 0.0f || ms < best_ms)) { best_ms = ms; best = plan; }
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (err != hipSuccess) return srt::from_hip(err);
  if (best_ms < 0.0f) return srtErrorNotSupported;   // no kernel qualifies: the caller's CPU path
  plan_cache().put(key_of(p), best);
  // leave `out` written by the chosen plan
  err = launch_plan(p, best, hs);
  if (chosen && chosenCapacity) std::snprintf(chosen, chosenCapacity, "%s", kPlanNames[best]);
  return srt::from_hip(err);
}

srtStatus srtPlanCacheClear(void) { plan_cache().clear(); return srtSuccess; }

srtStatus srtPlanCacheCount(size_t* count) {
  if (!count) return srtErrorInvalidValue;
  *count = plan_cache().size();
  return srtSuccess;
}

srtStatus srtPlanCacheSave(const char* path) { return path ? plan_cache().save(path) : srtErrorInvalidValue; }

srtStatus srtPlanCacheLoad(const char* path) { return path ? plan_cache().load(path) : srtErrorInvalidValue; }

}  // extern "C"
