//******************************************************************************
// matmul on the HIP platform: fills the role of platform/cuda/functions/CudaMatmul.swift, whose
// two functions always fall back to the cpu.  Written against include/srt_hip.h; not compiled
// in this environment (no Swift toolchain).
//******************************************************************************
import SwiftRTHip

//==============================================================================
// element type ids (role of StorageElement.swift:123-129 / CudaExtensions.swift type extensions)
extension Float { @inlinable public static var type: srtDataType { srtReal32F } }
extension Float16 { @inlinable public static var type: srtDataType { srtReal16F } }
extension BFloat16 { @inlinable public static var type: srtDataType { srtReal16BF } }
extension Double { @inlinable public static var type: srtDataType { srtReal64F } }

extension Order {
  /// role of `order.cublas` (CudaPlatform.swift:297-311); tiled orders have no native kernel
  @inlinable public var srt: srtOrder { self == .col ? srtOrderCol : srtOrderRow }
}

extension ActivationType {
  /// the native enum keeps this enum's case order (FunctionProperties.swift:44-51)
  @inlinable public var srt: srtActivation { srtActivation(rawValue: UInt32(rawValue)) }
}

//==============================================================================
// descriptors on the stack for the duration of one call (role of CudaExtensions.swift:24-84)
extension Tensor {
  @inlinable public func withTensor<Result>(
    using queue: HipQueue,
    _ body: (UnsafeRawPointer, UnsafePointer<srtTensorDescriptor>) -> Result
  ) -> Result {
    let data = deviceRead(using: queue)
    return shape.withUnsafePointer { s in
      strides.withUnsafePointer { st in
        logicalStrides.withUnsafePointer { ls in
          var d = srtTensorDescriptor(
            type: TensorElement.type, rank: UInt32(Shape.rank), order: order.srt,
            count: count, spanCount: spanCount, shape: s, strides: st, logicalStrides: ls)
          return withUnsafePointer(to: &d) { body(data, $0) }
        }
      }
    }
  }

  @inlinable public mutating func withMutableTensor<Result>(
    using queue: HipQueue,
    _ body: (UnsafeMutableRawPointer, UnsafePointer<srtTensorDescriptor>) -> Result
  ) -> Result {
    let data = deviceReadWrite(using: queue)
    return shape.withUnsafePointer { s in
      strides.withUnsafePointer { st in
        logicalStrides.withUnsafePointer { ls in
          var d = srtTensorDescriptor(
            type: TensorElement.type, rank: UInt32(Shape.rank), order: order.srt,
            count: count, spanCount: spanCount, shape: s, strides: st, logicalStrides: ls)
          return withUnsafePointer(to: &d) { body(data, $0) }
        }
      }
    }
  }
}

//==============================================================================
extension HipQueue {
  //--------------------------------------------------------------------------
  /// rank 2.  Same signature as CudaQueue.matmul (CudaMatmul.swift:25-29), so the operator in
  /// operators/Matmul.swift:29-45 and the pullbacks in MathDerivatives.swift:460-518 are unchanged.
  @inlinable func matmul<E>(
    _ lhs: TensorR2<E>, _ transposeLhs: Bool,
    _ rhs: TensorR2<E>, _ transposeRhs: Bool,
    _ result: inout TensorR2<E>
  ) where E.Value: Numeric {
    guard useGpu else { cpu_matmul(lhs, transposeLhs, rhs, transposeRhs, &result); return }
    diagnostic(.queueGpu, "matmul(\(lhs.name), transL: \(transposeLhs), \(rhs.name), transR: \(transposeRhs))",
               categories: .queueGpu)
    let status = result.withMutableTensor(using: self) { o, oDesc in
      lhs.withTensor(using: self) { a, aDesc in
        rhs.withTensor(using: self) { b, bDesc in
          srtMatmul(a, aDesc, transposeLhs ? 1 : 0, b, bDesc, transposeRhs ? 1 : 0, o, oDesc, stream)
        }
      }
    }
    cpuFallback(status) { $0.matmul(lhs, transposeLhs, rhs, transposeRhs, &result) }
  }

  //--------------------------------------------------------------------------
  /// rank 3 (batched).  Same signature as CudaMatmul.swift:44-48.
  @inlinable func matmul<E>(
    _ lhs: TensorR3<E>, _ transposeLhs: Bool,
    _ rhs: TensorR3<E>, _ transposeRhs: Bool,
    _ result: inout TensorR3<E>
  ) where E.Value: Numeric {
    guard useGpu else { cpu_matmul(lhs, transposeLhs, rhs, transposeRhs, &result); return }
    let status = result.withMutableTensor(using: self) { o, oDesc in
      lhs.withTensor(using: self) { a, aDesc in
        rhs.withTensor(using: self) { b, bDesc in
          srtMatmul(a, aDesc, transposeLhs ? 1 : 0, b, bDesc, transposeRhs ? 1 : 0, o, oDesc, stream)
        }
      }
    }
    cpuFallback(status) { $0.matmul(lhs, transposeLhs, rhs, transposeRhs, &result) }
  }

  //--------------------------------------------------------------------------
  /// Dense forward: activation(matmul + bias), fused in the GEMM epilogue.  New queue function:
  /// operators/Matmul.swift:57-72 (which drops its bias) calls this with `.identity`, and
  /// Dense.callAsFunction (SwiftRTLayers/Dense.swift:36-39) with the layer's activation.
  @inlinable func matmul<E>(
    _ lhs: TensorR2<E>, _ transposeLhs: Bool,
    _ rhs: TensorR2<E>, _ transposeRhs: Bool,
    bias: TensorR1<E>, activation: ActivationType, reluCeiling: Double = 0,
    _ result: inout TensorR2<E>
  ) where E.Value: Numeric {
    let status = result.withMutableTensor(using: self) { o, oDesc in
      lhs.withTensor(using: self) { a, aDesc in
        rhs.withTensor(using: self) { b, bDesc in
          bias.withTensor(using: self) { c, cDesc in
            srtMatmulBiasActivation(a, aDesc, transposeLhs ? 1 : 0, b, bDesc, transposeRhs ? 1 : 0,
                                    c, cDesc, activation.srt, reluCeiling, o, oDesc, stream)
          }
        }
      }
    }
    // no cpu op fuses the three steps; a caller without the native path composes
    // cpu_matmul, cpu_add and the activation as Recurrent.swift:157-161 does
    hipCheck(status)
  }
}

//==============================================================================
/// HipMatmul2: the retained-operation form (role of CudaMatmul2, CudaMatmul.swift:63-120, whose
/// `tune` is empty).  The first forward for a shape asks the native module to measure every kernel
/// plan the problem qualifies for; the winner is recorded in the module's plan cache under the
/// shape / layout / epilogue key, so this and every later matmul with that key run it.
public final class HipMatmul2<E>: DeviceMatmul2<E>
where E: StorageElement, E.Value: StorageElement & Numeric {
  public let queue: HipQueue
  public var tunedShapes = Set<[Int]>()

  @inlinable public init(queue: HipQueue) { self.queue = queue }

  @inlinable public override func forward(
    _ lhs: TensorR2<E>, _ transposeLhs: Bool,
    _ rhs: TensorR2<E>, _ transposeRhs: Bool,
    _ result: inout TensorR2<E>
  ) {
    let key = [lhs.shape[0], lhs.shape[1], rhs.shape[0], rhs.shape[1], transposeLhs ? 1 : 0, transposeRhs ? 1 : 0]
    if tunedShapes.insert(key).inserted {
      tune(lhs, transposeLhs, rhs, transposeRhs, &result)     // leaves `result` computed
    } else {
      queue.matmul(lhs, transposeLhs, rhs, transposeRhs, &result)
    }
  }

  @inlinable public func tune(
    _ lhs: TensorR2<E>, _ transposeLhs: Bool,
    _ rhs: TensorR2<E>, _ transposeRhs: Bool,
    _ result: inout TensorR2<E>
  ) {
    var name = [CChar](repeating: 0, count: 64)
    let status = result.withMutableTensor(using: queue) { o, oDesc in
      lhs.withTensor(using: queue) { a, aDesc in
        rhs.withTensor(using: queue) { b, bDesc in
          srtMatmulTune(a, aDesc, transposeLhs ? 1 : 0, b, bDesc, transposeRhs ? 1 : 0, nil, nil,
                        srtActivationIdentity, 0, o, oDesc, queue.stream, &name, 64)
        }
      }
    }
    cpuFallback(status) { $0.matmul(lhs, transposeLhs, rhs, transposeRhs, &result) }
    queue.diagnostic(.queueGpu, "matmul plan: \(String(cString: name))", categories: .queueGpu)
  }
}
