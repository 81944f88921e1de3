//******************************************************************************
// Element-wise queue functions and the Dense pullback on the HIP platform: the role of
// platform/cuda/functions/CudaMath.swift for the operations either side of matmul, and of
// platform/cuda/layers/CudaActivation.swift:101-127 for the activation gradient.
// Written against include/srt_hip.h; not compiled in this environment (no Swift toolchain).
//******************************************************************************
import SwiftRTHip

extension HipQueue {
  //--------------------------------------------------------------------------
  // tensor tensor.  Same shape of code as CudaQueue.add (CudaMath.swift:93-124): the flat entry
  // point when all three tensors are dense in one order, the strided one otherwise, and the
  // cpu function when the native module answers srtErrorNotSupported.
  @inlinable public func add<S, E>(
    _ lhs: Tensor<S, E>, _ rhs: Tensor<S, E>, _ out: inout Tensor<S, E>
  ) where E.Value: AdditiveArithmetic {
    assert(out.isContiguous, _messageElementsMustBeContiguous)
    guard useGpu else { cpu_add(lhs, rhs, &out); return }
    var status: srtStatus
    if canFlatten(lhs, rhs, out) {
      status = srtAddFlat(E.type, lhs.deviceRead(using: self), rhs.deviceRead(using: self),
                          out.deviceReadWrite(using: self), out.count, stream)
    } else {
      status = out.withMutableTensor(using: self) { o, oDesc in
        lhs.withTensor(using: self) { l, lDesc in
          rhs.withTensor(using: self) { r, rDesc in srtAdd(l, lDesc, r, rDesc, o, oDesc, stream) }
        }
      }
    }
    cpuFallback(status) { $0.add(lhs, rhs, &out) }
  }

  // tensor Element (CudaMath.swift:128-146)
  @inlinable public func add<S, E>(
    _ lhs: Tensor<S, E>, _ rhs: E.Value, _ out: inout Tensor<S, E>
  ) where E.Value: AdditiveArithmetic {
    guard useGpu else { cpu_add(lhs, rhs, &out); return }
    let element = E.stored(value: rhs)
    var status: srtStatus
    if canFlatten(lhs, out) {
      // dense operand and result: the flat tensor-element form (srtAddTEFlat, math_api.h:95-100)
      status = withUnsafePointer(to: element) {
        srtAddTEFlat(lhs.deviceRead(using: self), E.type, $0, out.deviceReadWrite(using: self), out.count, stream)
      }
    } else {
      status = out.withMutableTensor(using: self) { o, oDesc in
        lhs.withTensor(using: self) { l, lDesc in
          withUnsafePointer(to: element) { srtAddTE(l, lDesc, $0, o, oDesc, stream) }
        }
      }
    }
    cpuFallback(status) { $0.add(lhs, rhs, &out) }
  }

  //--------------------------------------------------------------------------
  // the remaining binary functions differ only in the entry point they name
  @inlinable func binary<S, E>(
    _ lhs: Tensor<S, E>, _ rhs: Tensor<S, E>, _ out: inout Tensor<S, E>,
    _ native: (UnsafeRawPointer, UnsafePointer<srtTensorDescriptor>, UnsafeRawPointer,
               UnsafePointer<srtTensorDescriptor>, UnsafeMutableRawPointer,
               UnsafePointer<srtTensorDescriptor>, srtStream?) -> srtStatus,
    _ fallback: (CpuQueue) -> Void
  ) {
    let status = out.withMutableTensor(using: self) { o, oDesc in
      lhs.withTensor(using: self) { l, lDesc in
        rhs.withTensor(using: self) { r, rDesc in native(l, lDesc, r, rDesc, o, oDesc, stream) }
      }
    }
    cpuFallback(status, fallback)
  }

  @inlinable public func subtract<S, E>(_ lhs: Tensor<S, E>, _ rhs: Tensor<S, E>, _ out: inout Tensor<S, E>)
  where E.Value: AdditiveArithmetic { binary(lhs, rhs, &out, srtSub) { $0.subtract(lhs, rhs, &out) } }

  @inlinable public func mul<S, E>(_ lhs: Tensor<S, E>, _ rhs: Tensor<S, E>, _ out: inout Tensor<S, E>)
  where E.Value: Numeric { binary(lhs, rhs, &out, srtMul) { $0.mul(lhs, rhs, &out) } }

  @inlinable public func div<S, E>(_ lhs: Tensor<S, E>, _ rhs: Tensor<S, E>, _ out: inout Tensor<S, E>)
  where E.Value: AlgebraicField { binary(lhs, rhs, &out, srtDiv) { $0.div(lhs, rhs, &out) } }

  @inlinable public func max<S, E>(_ lhs: Tensor<S, E>, _ rhs: Tensor<S, E>, _ out: inout Tensor<S, E>)
  where E.Value: Comparable { binary(lhs, rhs, &out, srtMax) { $0.max(lhs, rhs, &out) } }

  @inlinable public func min<S, E>(_ lhs: Tensor<S, E>, _ rhs: Tensor<S, E>, _ out: inout Tensor<S, E>)
  where E.Value: Comparable { binary(lhs, rhs, &out, srtMin) { $0.min(lhs, rhs, &out) } }

  //--------------------------------------------------------------------------
  // unary
  @inlinable func unary<S, E>(
    _ x: Tensor<S, E>, _ out: inout Tensor<S, E>,
    _ native: (UnsafeRawPointer, UnsafePointer<srtTensorDescriptor>, UnsafeMutableRawPointer,
               UnsafePointer<srtTensorDescriptor>, srtStream?) -> srtStatus,
    _ fallback: (CpuQueue) -> Void
  ) {
    let status = out.withMutableTensor(using: self) { o, oDesc in
      x.withTensor(using: self) { a, aDesc in native(a, aDesc, o, oDesc, stream) }
    }
    cpuFallback(status, fallback)
  }

  @inlinable public func neg<S, E>(_ x: Tensor<S, E>, _ out: inout Tensor<S, E>)
  where E.Value: SignedNumeric { unary(x, &out, srtNeg) { $0.neg(x, &out) } }

  @inlinable public func exp<S, E>(_ x: Tensor<S, E>, _ out: inout Tensor<S, E>)
  where E.Value: Real { unary(x, &out, srtExp) { $0.exp(x, &out) } }

  @inlinable public func sigmoid<S, E>(_ x: Tensor<S, E>, _ out: inout Tensor<S, E>)
  where E.Value: Real { unary(x, &out, srtSigmoid) { $0.sigmoid(x, &out) } }

  @inlinable public func tanh<S, E>(_ x: Tensor<S, E>, _ out: inout Tensor<S, E>)
  where E.Value: Real { unary(x, &out, srtTanh) { $0.tanh(x, &out) } }

  /// copy and cast: srtCopy converts between Float, Float16 and BFloat16 storage
  @inlinable public func copy<S, E, OE>(from x: Tensor<S, E>, to out: inout Tensor<S, OE>) {
    let status = out.withMutableTensor(using: self) { o, oDesc in
      x.withTensor(using: self) { a, aDesc in srtCopy(a, aDesc, o, oDesc, stream) }
    }
    cpuFallback(status) { $0.copy(from: x, to: &out) }
  }

  /// fill(_:with:) of a dense tensor (role of CudaFill.swift's srtFillFlat call)
  @inlinable public func fill<S, E>(_ out: inout Tensor<S, E>, with element: E.Value) {
    assert(out.isContiguous, _messageElementsMustBeContiguous)
    let stored = E.stored(value: element)
    let status = withUnsafePointer(to: stored) {
      srtFillFlat(E.type, out.deviceReadWrite(using: self), $0, out.count, stream)
    }
    cpuFallback(status) { $0.fill(&out, with: element) }
  }

  //--------------------------------------------------------------------------
  /// Pullback of the Dense epilogue: xDiff = yDiff * activation'(y), biasDiff = column sums of
  /// xDiff, in one pass.  Same roles as CudaActivation.backward(y:yDiff:x:xDiff:)
  /// (CudaActivation.swift:101-127; x is not needed: the derivative is taken through y) plus the
  /// bias term of _vjpMatmul(...bias:) that MathDerivatives.swift:520-554 leaves unimplemented.
  @inlinable public func activationBackward<E>(
    y: TensorR2<E>, yDiff: TensorR2<E>,
    activation: ActivationType, reluCeiling: Double = 0,
    xDiff: inout TensorR2<E>, biasDiff: inout TensorR1<E>
  ) where E.Value: Real {
    let status = xDiff.withMutableTensor(using: self) { dx, dxDesc in
      biasDiff.withMutableTensor(using: self) { db, dbDesc in
        y.withTensor(using: self) { yData, yDesc in
          yDiff.withTensor(using: self) { dy, dyDesc in
            srtActivationBackwardBias(yData, yDesc, dy, dyDesc, activation.srt, reluCeiling,
                                      dx, dxDesc, db, dbDesc, stream)
          }
        }
      }
    }
    hipCheck(status)
  }
}
