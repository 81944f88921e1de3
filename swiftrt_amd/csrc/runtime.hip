// Device, stream, event, memory and copy entry points of the C ABI (include/srt_hip.h).
// Thin, allocation-free wrappers over the HIP runtime, plus the stream-ordered caching
// device allocator that backs srtDeviceAllocate / srtDeviceFree.
#include <hip/hip_runtime.h>

#include <cstring>
#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "../../include/srt_hip.h"
#include "status.h"

namespace {

inline hipStream_t hs(srtStream s) { return reinterpret_cast<hipStream_t>(s); }
inline hipEvent_t he(srtEvent e) { return reinterpret_cast<hipEvent_t>(e); }

// ---- caching allocator ---------------------------------------------------------------------
// Blocks are binned by rounded size per device.  A free block remembers the stream it was last
// associated with; it is handed out again to the same stream at once (stream order protects it),
// to another stream only when an event recorded on the first stream has completed.  That event is
// recorded when the other stream first asks, not at free time: it then covers more work than it
// needs to, which is safe, and the common allocate / free / allocate cycle of one stream (a
// workspace per call) queues no event at all -- an event recorded after every free cost each such
// call about 5 us of idle device between its last kernel and the next call's first.
struct Block {
  void* ptr;
  size_t size;
  int device;
  hipStream_t stream;
  hipEvent_t ready;  // null while live and until another stream asks for the free block
  bool pending;      // free, possibly still in use by work queued on `stream`, no event recorded yet
};

const hipStream_t kNoStream = reinterpret_cast<hipStream_t>(~uintptr_t(0));   // matches no real stream

size_t round_size(size_t n) {
  if (n < 512) return 512;
  if (n <= (size_t(1) << 20)) {  // up to 1 MiB: next power of two
    size_t r = 512;
    while (r < n) r <<= 1;
    return r;
  }
  const size_t g = size_t(2) << 20;  // above: multiples of 2 MiB
  return (n + g - 1) / g * g;
}

class CachingAllocator {
 public:
  srtStatus allocate(void** out, size_t size, hipStream_t stream) {
    if (!out) return srtErrorInvalidValue;
    *out = nullptr;
    if (size == 0) return srtSuccess;
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return srtErrorNoDevice;
    const size_t rs = round_size(size);
    {
      std::lock_guard<std::mutex> lock(mu_);
      auto range = free_.equal_range(Key{device, rs});
      for (auto it = range.first; it != range.second; ++it) {
        Block& b = it->second;
        bool usable = (b.stream == stream);
        if (!usable && b.pending) {
          // first request from another stream: mark the point the block's stream has reached
          hipEvent_t ev = nullptr;
          if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) == hipSuccess &&
              hipEventRecord(ev, b.stream) == hipSuccess) {
            b.ready = ev;
            b.pending = false;
          } else {
            if (ev) (void)hipEventDestroy(ev);
            (void)hipGetLastError();
            continue;   // cannot be ordered now: leave it to its own stream
          }
        }
        if (!usable && b.ready) usable = (hipEventQuery(b.ready) == hipSuccess);
        if (!usable && !b.ready && !b.pending) usable = true;
        if (usable) {
          Block blk = b;
          free_.erase(it);
          if (blk.ready) { (void)hipEventDestroy(blk.ready); blk.ready = nullptr; }
          blk.pending = false;
          blk.stream = stream;
          live_[blk.ptr] = blk;
          *out = blk.ptr;
          return srtSuccess;
        }
      }
    }
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, rs);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      // give cached memory back to the driver and retry once
      empty_cache();
      e = hipMalloc(&p, rs);
      if (e != hipSuccess) { (void)hipGetLastError(); return srtErrorOutOfMemory; }
    }
    std::lock_guard<std::mutex> lock(mu_);
    live_[p] = Block{p, rs, device, stream, nullptr, false};
    *out = p;
    return srtSuccess;
  }

  srtStatus release(void* p) {
    if (!p) return srtSuccess;
    Block blk;
    {
      std::lock_guard<std::mutex> lock(mu_);
      auto it = live_.find(p);
      if (it == live_.end()) return srtErrorInvalidValue;
      blk = it->second;
      live_.erase(it);
    }
    blk.ready = nullptr;
    blk.pending = true;
    if (blk.stream == kNoStream) {
      // the stream was destroyed while the block was live: nothing can order the free, so make it
      // safe the slow way
      int prev = 0;
      (void)hipGetDevice(&prev);
      if (prev != blk.device) (void)hipSetDevice(blk.device);
      (void)hipDeviceSynchronize();
      if (prev != blk.device) (void)hipSetDevice(prev);
      blk.pending = false;
    }
    std::lock_guard<std::mutex> lock(mu_);
    free_.emplace(Key{blk.device, blk.size}, blk);
    return srtSuccess;
  }

  // Called before a stream is destroyed.  Its handle value may be given to a new stream later, so
  // cached blocks must not treat that stream as "the stream I was last used on"; and blocks still
  // live on it can no longer record an event there when they are freed (they fall back to a
  // device-wide synchronisation).
  void forget_stream(hipStream_t stream) {
    std::lock_guard<std::mutex> lock(mu_);
    for (auto& kv : free_) {
      Block& b = kv.second;
      if (b.stream != stream) continue;
      if (b.pending) {
        // last chance to order the block behind the stream's work: events outlive their stream
        int prev = 0;
        (void)hipGetDevice(&prev);
        if (prev != b.device) (void)hipSetDevice(b.device);
        hipEvent_t ev = nullptr;
        if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) == hipSuccess && hipEventRecord(ev, stream) == hipSuccess) {
          b.ready = ev;
        } else {
          if (ev) (void)hipEventDestroy(ev);
          (void)hipGetLastError();
          (void)hipStreamSynchronize(stream);
        }
        if (prev != b.device) (void)hipSetDevice(prev);
        b.pending = false;
      }
      b.stream = kNoStream;
    }
    for (auto& kv : live_)
      if (kv.second.stream == stream) kv.second.stream = kNoStream;
  }

  srtStatus empty_cache() {
    std::vector<Block> blocks;
    {
      std::lock_guard<std::mutex> lock(mu_);
      for (auto& kv : free_) blocks.push_back(kv.second);
      free_.clear();
    }
    int prev = 0;
    (void)hipGetDevice(&prev);
    for (Block& b : blocks) {
      (void)hipSetDevice(b.device);
      if (b.ready) { (void)hipEventSynchronize(b.ready); (void)hipEventDestroy(b.ready); }
      if (b.pending) (void)hipStreamSynchronize(b.stream);
      (void)hipFree(b.ptr);
    }
    (void)hipSetDevice(prev);
    return srtSuccess;
  }

 private:
  struct Key {
    int device;
    size_t size;
    bool operator<(const Key& o) const { return device != o.device ? device < o.device : size < o.size; }
  };
  std::mutex mu_;
  std::multimap<Key, Block> free_;
  std::unordered_map<void*, Block> live_;
};

CachingAllocator& allocator() {
  static CachingAllocator* a = new CachingAllocator();  // leaked on purpose: outlives HIP teardown
  return *a;
}

__global__ void fill_bytes_kernel(unsigned char* dst, unsigned char value, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) dst[i] = value;
}

__global__ void fill_words_kernel(uint32_t* dst, uint32_t value, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) dst[i] = value;
}

// Spins until `ticks` of the constant-rate wall clock have passed.  Exit is guaranteed: the
// clock always advances and ticks is bounded by the host.
__global__ void delay_kernel(unsigned long long ticks) {
  unsigned long long start = wall_clock64();
  while (wall_clock64() - start < ticks) { __builtin_amdgcn_s_sleep(32); }
}

}  // namespace

namespace srt {
void prepare_backward_scratch();   // activation_backward.hip
srtStatus from_hip(hipError_t e) {
  switch (e) {
    case hipSuccess: return srtSuccess;
    case hipErrorInvalidValue: return srtErrorInvalidValue;
    case hipErrorOutOfMemory: return srtErrorOutOfMemory;
    case hipErrorNotReady: return srtErrorNotReady;
    case hipErrorNotSupported: return srtErrorNotSupported;
    case hipErrorNoDevice:
    case hipErrorInvalidDevice: return srtErrorNoDevice;
    case hipErrorLaunchFailure:
    case hipErrorIllegalAddress:
    case hipErrorLaunchOutOfResources: return srtErrorLaunchFailure;
    default: (void)hipGetLastError(); return srtErrorUnknown;
  }
}
}  // namespace srt

using srt::from_hip;

extern "C" {

const char* srtGetStatusString(srtStatus status) {
  switch (status) {
    case srtSuccess: return "srtSuccess";
    case srtErrorInvalidValue: return "srtErrorInvalidValue";
    case srtErrorOutOfMemory: return "srtErrorOutOfMemory";
    case srtErrorNotReady: return "srtErrorNotReady";
    case srtErrorNotSupported: return "srtErrorNotSupported";
    case srtErrorLaunchFailure: return "srtErrorLaunchFailure";
    case srtErrorNoDevice: return "srtErrorNoDevice";
    default: return "srtErrorUnknown";
  }
}

int32_t srtGetVersion(void) { return 100; }

srtStatus srtGetDeviceCount(int32_t* count) {
  if (!count) return srtErrorInvalidValue;
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess) { (void)hipGetLastError(); *count = 0; return srtErrorNoDevice; }
  *count = n;
  return srtSuccess;
}

srtStatus srtSetDevice(int32_t device) { return from_hip(hipSetDevice(device)); }

srtStatus srtGetDevice(int32_t* device) {
  if (!device) return srtErrorInvalidValue;
  int d = 0;
  hipError_t e = hipGetDevice(&d);
  *device = d;
  return from_hip(e);
}

srtStatus srtGetDeviceProperties(srtDeviceProperties* props, int32_t device) {
  if (!props) return srtErrorInvalidValue;
  hipDeviceProp_t p;
  hipError_t e = hipGetDeviceProperties(&p, device);
  if (e != hipSuccess) return from_hip(e);
  std::memset(props, 0, sizeof(*props));
  std::strncpy(props->name, p.name, sizeof(props->name) - 1);
  std::strncpy(props->archName, p.gcnArchName, sizeof(props->archName) - 1);
  props->totalGlobalMem = p.totalGlobalMem;
  props->multiProcessorCount = p.multiProcessorCount;
  props->clockRateKHz = p.clockRate;
  props->memoryClockRateKHz = p.memoryClockRate;
  props->memoryBusWidthBits = p.memoryBusWidth;
  props->l2CacheBytes = p.l2CacheSize;
  props->sharedMemPerBlockBytes = (int32_t)p.maxSharedMemoryPerMultiProcessor;
  props->warpSize = p.warpSize;
  return srtSuccess;
}

srtStatus srtDeviceSynchronize(void) { return from_hip(hipDeviceSynchronize()); }

srtStatus srtStreamCreate(srtStream* stream) {
  if (!stream) return srtErrorInvalidValue;
  hipStream_t s = nullptr;
  hipError_t e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);  // default priority
  *stream = reinterpret_cast<srtStream>(s);
  // once per device: the address of the fixed workspace of srtActivationBackwardBiasNoAlloc
  if (e == hipSuccess) srt::prepare_backward_scratch();
  return from_hip(e);
}

srtStatus srtStreamDestroy(srtStream stream) {
  if (!stream) return srtSuccess;
  allocator().forget_stream(hs(stream));
  return from_hip(hipStreamDestroy(hs(stream)));
}

srtStatus srtStreamSynchronize(srtStream stream) { return from_hip(hipStreamSynchronize(hs(stream))); }

srtStatus srtEventCreate(srtEvent* event, int32_t enableTiming) {
  if (!event) return srtErrorInvalidValue;
  hipEvent_t e = nullptr;
  hipError_t r = hipEventCreateWithFlags(&e, enableTiming ? hipEventDefault : hipEventDisableTiming);
  *event = reinterpret_cast<srtEvent>(e);
  return from_hip(r);
}

srtStatus srtEventDestroy(srtEvent event) {
  if (!event) return srtSuccess;
  return from_hip(hipEventDestroy(he(event)));
}

srtStatus srtEventRecord(srtEvent event, srtStream stream) {
  if (!event) return srtErrorInvalidValue;
  return from_hip(hipEventRecord(he(event), hs(stream)));
}

srtStatus srtStreamWaitEvent(srtStream stream, srtEvent event) {
  if (!event) return srtErrorInvalidValue;
  return from_hip(hipStreamWaitEvent(hs(stream), he(event), 0));
}

srtStatus srtEventSynchronize(srtEvent event) {
  if (!event) return srtErrorInvalidValue;
  return from_hip(hipEventSynchronize(he(event)));
}

srtStatus srtEventQuery(srtEvent event) {
  if (!event) return srtErrorInvalidValue;
  hipError_t e = hipEventQuery(he(event));
  if (e == hipErrorNotReady) { (void)hipGetLastError(); return srtErrorNotReady; }
  return from_hip(e);
}

srtStatus srtEventElapsedTime(float* milliseconds, srtEvent start, srtEvent stop) {
  if (!milliseconds || !start || !stop) return srtErrorInvalidValue;
  return from_hip(hipEventElapsedTime(milliseconds, he(start), he(stop)));
}

srtStatus srtDeviceAllocate(void** devPtr, size_t size, srtStream stream) {
  return allocator().allocate(devPtr, size, hs(stream));
}

srtStatus srtDeviceFree(void* devPtr) { return allocator().release(devPtr); }

srtStatus srtDeviceEmptyCache(void) { return allocator().empty_cache(); }

srtStatus srtHostAllocate(void** hostPtr, size_t size) {
  if (!hostPtr) return srtErrorInvalidValue;
  *hostPtr = nullptr;
  if (size == 0) return srtSuccess;
  hipError_t e = hipHostMalloc(hostPtr, size, hipHostMallocDefault);
  if (e != hipSuccess) { (void)hipGetLastError(); return srtErrorOutOfMemory; }
  return srtSuccess;
}

srtStatus srtHostFree(void* hostPtr) {
  if (!hostPtr) return srtSuccess;
  return from_hip(hipHostFree(hostPtr));
}

srtStatus srtMemcpyAsync(void* dst, const void* src, size_t byteCount, srtMemcpyKind kind, srtStream stream) {
  if (byteCount == 0) return srtSuccess;
  if (!dst || !src) return srtErrorInvalidValue;
  hipMemcpyKind k;
  switch (kind) {
    case srtMemcpyHostToDevice: k = hipMemcpyHostToDevice; break;
    case srtMemcpyDeviceToHost: k = hipMemcpyDeviceToHost; break;
    case srtMemcpyDeviceToDevice: k = hipMemcpyDeviceToDevice; break;
    default: return srtErrorInvalidValue;
  }
  return from_hip(hipMemcpyAsync(dst, src, byteCount, k, hs(stream)));
}

srtStatus srtMemsetAsync(void* dst, int32_t value, size_t byteCount, srtStream stream) {
  if (byteCount == 0) return srtSuccess;
  if (!dst) return srtErrorInvalidValue;
  const unsigned char v = (unsigned char)value;
  if ((reinterpret_cast<uintptr_t>(dst) & 3u) == 0 && (byteCount & 3u) == 0) {
    const size_t words = byteCount / 4;
    const uint32_t w = 0x01010101u * v;
    size_t blocks = (words + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(fill_words_kernel, dim3((unsigned)blocks), dim3(256), 0, hs(stream),
                       reinterpret_cast<uint32_t*>(dst), w, words);
  } else {
    size_t blocks = (byteCount + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(fill_bytes_kernel, dim3((unsigned)blocks), dim3(256), 0, hs(stream),
                       reinterpret_cast<unsigned char*>(dst), v, byteCount);
  }
  return from_hip(srt::launch_status(hs(stream)));
}

srtStatus srtDelayStream(double seconds, srtStream stream) {
  if (!(seconds >= 0.0)) return srtErrorInvalidValue;
  if (seconds > 10.0) seconds = 10.0;
  int device = 0, rate_khz = 0;
  if (hipGetDevice(&device) != hipSuccess) return srtErrorNoDevice;
  if (hipDeviceGetAttribute(&rate_khz, hipDeviceAttributeWallClockRate, device) != hipSuccess || rate_khz <= 0) {
    (void)hipGetLastError();
    rate_khz = 100000;  // 100 MHz constant clock
  }
  unsigned long long ticks = (unsigned long long)(seconds * 1000.0 * (double)rate_khz);
  hipLaunchKernelGGL(delay_kernel, dim3(1), dim3(1), 0, hs(stream), ticks);
  return from_hip(hipGetLastError());
}

}  // extern "C"
