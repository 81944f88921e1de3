// Header-only C++ mirror, above the C ABI (include/srt_hip.h), of the host types the reference
// implements in Swift for this path: HipQueue / HipDeviceMemory / HipEvent in the roles of
// platform/cuda/device/CudaQueue.swift, CudaDevice.swift:96-162 and CudaEvent.swift, a Tensor
// carrying shape / strides / order with a host and a device replica (tensor/Tensor.swift:26-54,
// platform/common/DiscreteStorage.swift:211-381), the matmul operators
// (operators/Matmul.swift:29-72) and Dense (SwiftRTLayers/Dense.swift:21-71).
// No arithmetic lives here: every operation is a call into the native module.  A status of
// srtErrorNotSupported is thrown as NotSupported (a Swift caller would run its cpu_matmul).
#pragma once
#include <cstdint>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/srt_hip.h"

namespace srt_host {

struct Error : std::runtime_error {
  srtStatus status;
  Error(srtStatus s, const std::string& what) : std::runtime_error(what + ": " + srtGetStatusString(s)), status(s) {}
};
struct NotSupported : Error {
  using Error::Error;
};

// role of cudaCheck / cpuFallback's split (CudaPlatform.swift:122-193)
inline void check(srtStatus s, const char* what) {
  if (s == srtSuccess) return;
  if (s == srtErrorNotSupported) throw NotSupported(s, what);
  throw Error(s, what);
}

class HipQueue;

class HipDeviceMemory {
 public:
  HipDeviceMemory(size_t bytes, srtStream stream) : bytes_(bytes), stream_(stream), last_stream_(stream) {
    size_t padded = (bytes + 31) / 32 * 32;   // CudaDevice.swift:141-142
    check(srtDeviceAllocate(&ptr_, padded ? padded : 32, stream), "srtDeviceAllocate");
  }
  // The free hands the block back to the allocating stream at once: work another stream still has in
  // flight on it is ordered first (event on that stream, wait on the allocating one).
  ~HipDeviceMemory() {
    if (last_stream_ != stream_) {
      srtEvent e = nullptr;
      if (srtEventCreate(&e, 0) == srtSuccess) {
        if (srtEventRecord(e, last_stream_) == srtSuccess) (void)srtStreamWaitEvent(stream_, e);
        (void)srtEventDestroy(e);
      }
    }
    srtDeviceFree(ptr_);
  }
  void used_on(srtStream stream) { last_stream_ = stream; }
  HipDeviceMemory(const HipDeviceMemory&) = delete;
  HipDeviceMemory& operator=(const HipDeviceMemory&) = delete;
  void* pointer() const { return ptr_; }
  size_t byte_count() const { return bytes_; }

 private:
  void* ptr_ = nullptr;
  size_t bytes_;
  srtStream stream_, last_stream_;
};

class HipEvent {
 public:
  explicit HipEvent(bool timing = false) { check(srtEventCreate(&e_, timing ? 1 : 0), "srtEventCreate"); }
  ~HipEvent() { srtEventDestroy(e_); }
  HipEvent(const HipEvent&) = delete;
  srtEvent handle() const { return e_; }
  void wait() const { check(srtEventSynchronize(e_), "srtEventSynchronize"); }
  bool occurred() const { return srtEventQuery(e_) == srtSuccess; }

 private:
  srtEvent e_ = nullptr;
};

enum class Order { col = srtOrderCol, row = srtOrderRow };
enum class ActivationType { sigmoid, relu, tanh, clippedRelu, elu, identity };   // FunctionProperties.swift:44-51

template <typename E> struct ElementType;
template <> struct ElementType<float> { static constexpr srtDataType type = srtReal32F; };
struct Float16 { uint16_t bits; };
struct BFloat16 { uint16_t bits; };
template <> struct ElementType<Float16> { static constexpr srtDataType type = srtReal16F; };
template <> struct ElementType<BFloat16> { static constexpr srtDataType type = srtReal16BF; };

class HipQueue {
 public:
  explicit HipQueue(int gpu = 0) : gpu_(gpu) {
    check(srtSetDevice(gpu), "srtSetDevice");
    check(srtStreamCreate(&stream_), "srtStreamCreate");
  }
  ~HipQueue() { srtStreamDestroy(stream_); }
  HipQueue(const HipQueue&) = delete;
  srtStream stream() const { return stream_; }
  std::shared_ptr<HipDeviceMemory> allocate(size_t bytes) { return std::make_shared<HipDeviceMemory>(bytes, stream_); }
  void copy_to_device(void* dst, const void* src, size_t n) {
    check(srtMemcpyAsync(dst, src, n, srtMemcpyHostToDevice, stream_), "srtMemcpyAsync");
  }
  void copy_to_host(void* dst, const void* src, size_t n) {
    check(srtMemcpyAsync(dst, src, n, srtMemcpyDeviceToHost, stream_), "srtMemcpyAsync");
  }
  void record(HipEvent& e) { check(srtEventRecord(e.handle(), stream_), "srtEventRecord"); }
  void wait(const HipEvent& e) { check(srtStreamWaitEvent(stream_, e.handle()), "srtStreamWaitEvent"); }
  void wait_for_completion() { check(srtStreamSynchronize(stream_), "srtStreamSynchronize"); }

 private:
  int gpu_;
  srtStream stream_ = nullptr;
};

// Tensor<E>: rank 1..3, shape + strides over shared storage with lazily migrated replicas.
template <typename E>
class Tensor {
  struct Storage {
    std::vector<E> host;
    std::shared_ptr<HipDeviceMemory> device;
    int host_version = 0, device_version = -1;
    HipQueue* last_queue = nullptr;
  };

 public:
  Tensor(std::vector<size_t> shape, Order order = Order::row) : shape_(std::move(shape)), order_(order) {
    size_t n = 1;
    for (size_t s : shape_) n *= s;
    storage_ = std::make_shared<Storage>();
    storage_->host.resize(n);
    strides_.assign(shape_.size(), 1);
    for (int i = (int)shape_.size() - 2; i >= 0; --i) strides_[i] = strides_[i + 1] * shape_[i + 1];
    const size_t r = shape_.size();
    if (order == Order::col && r >= 2) { strides_[r - 2] = 1; strides_[r - 1] = shape_[r - 2]; }
  }
  Tensor(std::vector<size_t> shape, const std::vector<E>& values, Order order = Order::row) : Tensor(shape, order) {
    // values are given in logical row-major order
    const size_t r = shape_.size();
    if (order == Order::col && r >= 2) {
      const size_t rows = shape_[r - 2], cols = shape_[r - 1], mats = values.size() / (rows * cols);
      for (size_t b = 0; b < mats; ++b)
        for (size_t i = 0; i < rows; ++i)
          for (size_t j = 0; j < cols; ++j) storage_->host[b * rows * cols + j * rows + i] = values[b * rows * cols + i * cols + j];
    } else {
      storage_->host = values;
    }
  }

  const std::vector<size_t>& shape() const { return shape_; }
  const std::vector<size_t>& strides() const { return strides_; }
  Order order() const { return order_; }
  size_t rank() const { return shape_.size(); }

  // `.t`: zero-copy swap of the last two extents and strides (TensorInit.swift:844-890)
  Tensor t() const {
    Tensor v = *this;
    const size_t r = rank();
    std::swap(v.shape_[r - 1], v.shape_[r - 2]);
    std::swap(v.strides_[r - 1], v.strides_[r - 2]);
    return v;
  }

  // role of Tensor.deviceRead / deviceReadWrite (Tensor.swift:558-582)
  const void* device_read(HipQueue& q) const { return migrate(q); }
  void* device_read_write(HipQueue& q) {
    void* p = migrate(q);
    storage_->device_version = std::max(storage_->device_version, storage_->host_version) + 1;
    return p;
  }

  // logical values in row-major order, synchronising device -> host first when needed
  std::vector<E> values() const {
    Storage& s = *storage_;
    if (s.device && s.device_version > s.host_version) {
      s.last_queue->copy_to_host(s.host.data(), s.device->pointer(), s.host.size() * sizeof(E));
      s.last_queue->wait_for_completion();
      s.host_version = s.device_version;
    }
    size_t n = 1;
    for (size_t d : shape_) n *= d;
    std::vector<E> out(n);
    std::vector<size_t> idx(rank(), 0);
    for (size_t i = 0; i < n; ++i) {
      size_t off = offset_;
      for (size_t d = 0; d < rank(); ++d) off += idx[d] * strides_[d];
      out[i] = s.host[off];
      for (int d = (int)rank() - 1; d >= 0; --d) {
        if (++idx[d] < shape_[d]) break;
        idx[d] = 0;
      }
    }
    return out;
  }

  // descriptor for the duration of one call (role of Tensor.withTensor, CudaExtensions.swift:24-84)
  srtTensorDescriptor descriptor() const {
    size_t count = 1, span = 1;
    for (size_t d = 0; d < rank(); ++d) { count *= shape_[d]; span += (shape_[d] ? shape_[d] - 1 : 0) * strides_[d]; }
    return srtTensorDescriptor{ElementType<E>::type, (uint32_t)rank(), (srtOrder)order_, count, count ? span : 0,
                               shape_.data(), strides_.data(), strides_.data()};
  }

 private:
  void* migrate(HipQueue& q) const {
    Storage& s = *storage_;
    if (!s.device) s.device = q.allocate(s.host.size() * sizeof(E));
    if (s.last_queue && s.last_queue != &q) {   // cross-queue ordering through an event
      HipEvent e;
      s.last_queue->record(e);
      q.wait(e);
    }
    s.last_queue = &q;
    s.device->used_on(q.stream());
    if (s.device_version < s.host_version) {
      q.copy_to_device(s.device->pointer(), s.host.data(), s.host.size() * sizeof(E));
      q.wait_for_completion();
      s.device_version = s.host_version;
    }
    return static_cast<char*>(s.device->pointer()) + offset_ * sizeof(E);
  }

  std::vector<size_t> shape_, strides_;
  size_t offset_ = 0;
  Order order_;
  std::shared_ptr<Storage> storage_;
};

// role of HipQueue.matmul (CudaMatmul.swift:25-61) for rank 2 and rank 3
template <typename E>
void queue_matmul(HipQueue& q, const Tensor<E>& lhs, bool tl, const Tensor<E>& rhs, bool tr, Tensor<E>& result,
                  const Tensor<E>* bias = nullptr, ActivationType act = ActivationType::identity, double coef = 0.0) {
  const void* a = lhs.device_read(q);
  const void* b = rhs.device_read(q);
  const void* c = bias ? bias->device_read(q) : nullptr;
  void* o = result.device_read_write(q);
  srtTensorDescriptor ad = lhs.descriptor(), bd = rhs.descriptor(), od = result.descriptor(), cd{};
  if (bias) cd = bias->descriptor();
  check(srtMatmulBiasActivation(a, &ad, tl, b, &bd, tr, c, bias ? &cd : nullptr, (srtActivation)act, coef, o, &od,
                                q.stream()),
        "srtMatmul");
}

// matmul(_:transposed:_:transposed:[bias:]) (operators/Matmul.swift:29-72); result dense in lhs.order
template <typename E>
Tensor<E> matmul(HipQueue& q, const Tensor<E>& lhs, bool transposed_lhs, const Tensor<E>& rhs, bool transposed_rhs,
                 const Tensor<E>* bias = nullptr) {
  std::vector<size_t> ls = lhs.shape(), rs = rhs.shape();
  const size_t r = ls.size();
  if (r != rs.size() || r < 2 || r > 3) throw std::invalid_argument("matmul takes two rank-2 or two rank-3 tensors");
  if (transposed_lhs) std::swap(ls[r - 1], ls[r - 2]);
  if (transposed_rhs) std::swap(rs[r - 1], rs[r - 2]);
  if (ls[r - 1] != rs[r - 2]) throw std::invalid_argument("matmul inner dimensions must be equal");
  std::vector<size_t> os(ls.begin(), ls.end() - 1);
  os.push_back(rs[r - 1]);
  Tensor<E> result(os, lhs.order());
  queue_matmul(q, lhs, transposed_lhs, rhs, transposed_rhs, result, bias);
  return result;
}

// Dense<S,E> (SwiftRTLayers/Dense.swift:21-71): activation(matmul(input, weight) + bias), one fused call
template <typename E>
struct Dense {
  Tensor<E> weight, bias;
  ActivationType activation;
  double coef = 0.0;
  Tensor<E> operator()(HipQueue& q, const Tensor<E>& x) const {
    if (x.shape()[1] != weight.shape()[0]) throw std::invalid_argument("matmul inner dimensions must be equal");
    Tensor<E> result({x.shape()[0], weight.shape()[1]}, x.order());
    queue_matmul(q, x, false, weight, false, result, &bias, activation, coef);
    return result;
  }
};

// ---- element-wise neighbours (role of CudaQueue.add / mul / max / sigmoid / tanh ...,
// platform/cuda/functions/CudaMath.swift:93-150) -----------------------------------------------------
using BinaryFn = srtStatus (*)(const void*, const srtTensorDescriptor*, const void*, const srtTensorDescriptor*,
                               void*, const srtTensorDescriptor*, srtStream);
using ElementFn = srtStatus (*)(const void*, const srtTensorDescriptor*, const void*, void*,
                                const srtTensorDescriptor*, srtStream);
using UnaryFn = srtStatus (*)(const void*, const srtTensorDescriptor*, void*, const srtTensorDescriptor*, srtStream);

template <typename E>
Tensor<E> binary(HipQueue& q, BinaryFn fn, const Tensor<E>& lhs, const Tensor<E>& rhs, const char* what) {
  if (lhs.shape() != rhs.shape()) throw std::invalid_argument("element-wise operands must have one shape");
  Tensor<E> out(lhs.shape(), lhs.order());
  const void* a = lhs.device_read(q);
  const void* b = rhs.device_read(q);
  void* o = out.device_read_write(q);
  srtTensorDescriptor ad = lhs.descriptor(), bd = rhs.descriptor(), od = out.descriptor();
  check(fn(a, &ad, b, &bd, o, &od, q.stream()), what);
  return out;
}

template <typename E>
Tensor<E> binary_element(HipQueue& q, ElementFn fn, const Tensor<E>& lhs, E element, const char* what) {
  Tensor<E> out(lhs.shape(), lhs.order());
  const void* a = lhs.device_read(q);
  void* o = out.device_read_write(q);
  srtTensorDescriptor ad = lhs.descriptor(), od = out.descriptor();
  check(fn(a, &ad, &element, o, &od, q.stream()), what);
  return out;
}

template <typename E>
Tensor<E> unary(HipQueue& q, UnaryFn fn, const Tensor<E>& x, const char* what) {
  Tensor<E> out(x.shape(), x.order());
  const void* a = x.device_read(q);
  void* o = out.device_read_write(q);
  srtTensorDescriptor ad = x.descriptor(), od = out.descriptor();
  check(fn(a, &ad, o, &od, q.stream()), what);
  return out;
}

template <typename E> Tensor<E> add(HipQueue& q, const Tensor<E>& a, const Tensor<E>& b) { return binary(q, srtAdd, a, b, "srtAdd"); }
template <typename E> Tensor<E> mul(HipQueue& q, const Tensor<E>& a, const Tensor<E>& b) { return binary(q, srtMul, a, b, "srtMul"); }
template <typename E> Tensor<E> add(HipQueue& q, const Tensor<E>& a, E e) { return binary_element(q, srtAddTE, a, e, "srtAddTE"); }
template <typename E> Tensor<E> relu(HipQueue& q, const Tensor<E>& a) { return binary_element(q, srtMaxTE, a, E{}, "srtMaxTE"); }
template <typename E> Tensor<E> sigmoid(HipQueue& q, const Tensor<E>& a) { return unary(q, srtSigmoid, a, "srtSigmoid"); }
template <typename E> Tensor<E> tanh(HipQueue& q, const Tensor<E>& a) { return unary(q, srtTanh, a, "srtTanh"); }

// ---- backward of Dense: (dx, dweight, dbias) for y = layer(x) and the gradient of y ------------------
// dz and dbias come from one fused pass (role of CudaActivation.backward,
// platform/cuda/layers/CudaActivation.swift:101-127, plus the bias pullback the reference leaves as
// fatalError, MathDerivatives.swift:520-554); dx = dz W^T, dW = x^T dz (matmulGradients :460-482).
template <typename E>
struct DenseGradients { Tensor<E> dx, dweight, dbias; };

template <typename E>
DenseGradients<E> dense_backward(HipQueue& q, const Dense<E>& layer, const Tensor<E>& x, const Tensor<E>& y,
                                 const Tensor<E>& out_grad) {
  Tensor<E> dz(y.shape(), y.order()), dbias({y.shape()[1]});
  const void* yp = y.device_read(q);
  const void* gp = out_grad.device_read(q);
  void* zp = dz.device_read_write(q);
  void* bp = dbias.device_read_write(q);
  srtTensorDescriptor yd = y.descriptor(), gd = out_grad.descriptor(), zd = dz.descriptor(), bd = dbias.descriptor();
  check(srtActivationBackwardBias(yp, &yd, gp, &gd, (srtActivation)layer.activation, layer.coef, zp, &zd, bp, &bd,
                                  q.stream()),
        "srtActivationBackwardBias");
  return DenseGradients<E>{matmul(q, dz, false, layer.weight, true), matmul(q, x, true, dz, false), dbias};
}

}  // namespace srt_host
