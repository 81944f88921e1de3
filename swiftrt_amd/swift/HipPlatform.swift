//******************************************************************************
// HIP platform for SwiftRT (MI355X / gfx950).
//
// Drop these files into Sources/SwiftRTCore/platform/hip/ and add, beside the existing
// selection in platform/common/Platform.swift:21-25,
//
//     #if canImport(SwiftRTHip)
//     public typealias Platform = HipPlatform
//     #elseif canImport(SwiftRTCuda) ...
//
// Types here fill the roles of platform/cuda/device/{CudaPlatform,CudaDevice,CudaQueue,
// CudaEvent}.swift.  They were written against include/srt_hip.h; this environment has no
// Swift toolchain, so they have not been compiled.
//******************************************************************************
import Foundation
import SwiftRTHip

//==============================================================================
/// hipCheck: role of cudaCheck (CudaPlatform.swift:180-193).  Any status other than success
/// is a hard error: report and trap.
@inlinable public func hipCheck(
  _ status: srtStatus, file: String = #file, function: String = #function, line: Int = #line
) {
  if status != srtSuccess {
    let name = String(cString: srtGetStatusString(status))
    _ = srtDeviceSynchronize()
    fatalError("hip error \(name) in \(function) at \(file):\(line)")
  }
}

//==============================================================================
/// HipPlatform: role of CudaPlatform (CudaPlatform.swift:22-115)
public final class HipPlatform: ComputePlatform {
  public typealias Storage = DiscreteStorage
  public static var local = HipPlatform()
  public static var acceleratorQueueCount: Int = 2
  public static let startTime = Date()

  public var discreteMemoryDeviceId: Int { 1 }
  public var devices: [HipDevice]
  public let name: String
  @inlinable public static var queueStack: [HipQueue] {
    get { local.queueStack } set { local.queueStack = newValue }
  }
  public var queueStack: [HipQueue]

  @inlinable public init(name: String? = nil) {
    self.name = name ?? "\(Self.self)"
    // device 0 is the cpu, as in the reference's numbering
    let cpuDevice = HipDevice(index: 0)
    devices = [cpuDevice]
    var gpuCount: Int32 = 0
    hipCheck(srtGetDeviceCount(&gpuCount))
    for i in 1..<Int(gpuCount + 1) { devices.append(HipDevice(index: i)) }
    // the first gpu queue (or the cpu queue when no gpu is visible) is the default
    let defaultDevice = gpuCount > 0 ? 1 : 0
    queueStack = [devices[defaultDevice].queues[0]]
  }

  /// cpuFallback: role of CudaPlatform.swift:122-144.  srtErrorNotSupported means the native
  /// module declined the layout or element type; run the same op on the cpu queue instead.
  @inlinable public static func cpuFallback(_ status: srtStatus, _ body: (HipQueue) -> Void) {
    if status == srtErrorNotSupported {
      using(device: 0) { body(currentQueue) }
    } else {
      hipCheck(status)
    }
  }
}

//==============================================================================
/// HipDevice: role of CudaDevice (CudaDevice.swift:22-94)
public final class HipDevice: ComputeDevice {
  public let index: Int
  public let memoryType: MemoryType
  public let name: String
  public var queues: [HipQueue]
  public var properties: [String]

  @inlinable public init(index: Int) {
    let isCpu = index == 0
    self.index = index
    self.name = isCpu ? "cpu:0" : "gpu:\(index - 1)"
    self.memoryType = isCpu ? .unified : .discrete
    properties = []
    queues = []
    if isCpu {
      queues.append(HipQueue(deviceIndex: index, name: "\(name)_q0", queueMode: .sync, useGpu: false))
    } else {
      var p = srtDeviceProperties()
      hipCheck(srtGetDeviceProperties(&p, Int32(index - 1)))
      let gpu = withUnsafePointer(to: &p.name) {
        $0.withMemoryRebound(to: CChar.self, capacity: 256) { String(cString: $0) }
      }
      properties = ["[type: \(gpu), multiprocessors: \(p.multiProcessorCount), "
        + "memory: \(p.totalGlobalMem >> 30) GB, addressing: \(memoryType)]"]
      for i in 0..<HipPlatform.acceleratorQueueCount {
        queues.append(HipQueue(deviceIndex: index, name: "\(name)_q\(i)", queueMode: .async, useGpu: true))
      }
    }
  }

  @inlinable public func select() { hipCheck(srtSetDevice(Int32(index - 1))) }
}

//==============================================================================
/// HipDeviceMemory: role of CudaDeviceMemory (CudaDevice.swift:96-162).  The Swift object
/// owns the pointer; the native module keeps no reference to tensor memory.
public final class HipDeviceMemory: DeviceMemory {
  public let buffer: UnsafeMutableRawBufferPointer
  public let deviceIndex: Int
  public var name: String?
  public var releaseMessage: String?
  public let type: MemoryType
  public var version: Int
  public let isReference: Bool

  @inlinable public var mutablePointer: UnsafeMutableRawPointer { UnsafeMutableRawPointer(buffer.baseAddress!) }
  @inlinable public var pointer: UnsafeRawPointer { UnsafeRawPointer(buffer.baseAddress!) }

  @inlinable public init(_ deviceIndex: Int, _ byteCount: Int, _ stream: srtStream?) {
    self.deviceIndex = deviceIndex
    // pad to the widest vector access, as CudaDevice.swift:141-142 does
    let padded = roundUp(byteCount, multiple: 32)
    var p: UnsafeMutableRawPointer?
    hipCheck(srtDeviceAllocate(&p, padded, stream))
    buffer = UnsafeMutableRawBufferPointer(start: p, count: byteCount)
    type = .discrete
    version = -1
    isReference = false
  }

  @inlinable deinit { if !isReference { hipCheck(srtDeviceFree(buffer.baseAddress!)) } }
}

//==============================================================================
/// HipEvent: role of CudaEvent (CudaEvent.swift:23-75)
public final class HipEvent: QueueEvent {
  public let handle: srtEvent
  public var recordedTime: Date?

  @inlinable public init(options: QueueEventOptions) {
    var e: srtEvent?
    hipCheck(srtEventCreate(&e, options.contains(.timing) ? 1 : 0))
    handle = e!
  }
  @inlinable deinit { _ = srtEventDestroy(handle) }
  @inlinable public var occurred: Bool { srtEventQuery(handle) == srtSuccess }
  @inlinable public func wait() { hipCheck(srtEventSynchronize(handle)) }
}

//==============================================================================
/// HipQueue: role of CudaQueue (CudaQueue.swift:22-196): one non-blocking stream on one device.
public final class HipQueue: DeviceQueue, CpuFunctions {
  public let creatorThread: Thread
  public var defaultQueueEventOptions: QueueEventOptions
  public let deviceIndex: Int
  public let id: Int
  public let memoryType: MemoryType
  public let mode: DeviceQueueMode
  public let name: String
  public let queue: DispatchQueue
  public let group: DispatchGroup
  public let useGpu: Bool
  public let gpuId: Int
  public let stream: srtStream?
  @inlinable public var usesCpu: Bool { !useGpu }

  @inlinable public init(deviceIndex: Int, name: String, queueMode: DeviceQueueMode, useGpu: Bool) {
    self.id = Platform.queueId.next
    self.name = name
    self.deviceIndex = deviceIndex
    self.gpuId = Swift.max(0, deviceIndex - 1)
    self.creatorThread = Thread.current
    self.defaultQueueEventOptions = QueueEventOptions()
    self.memoryType = useGpu ? .discrete : .unified
    self.mode = queueMode
    self.queue = DispatchQueue(label: name)
    self.group = DispatchGroup()
    self.useGpu = useGpu
    if useGpu {
      hipCheck(srtSetDevice(Int32(gpuId)))
      var s: srtStream?
      hipCheck(srtStreamCreate(&s))     // non-blocking, default priority
      stream = s
    } else {
      stream = nil
    }
  }

  @inlinable public func allocate(byteCount: Int, heapIndex: Int = 0) -> DeviceMemory {
    if usesCpu { return CpuDeviceMemory(deviceIndex, byteCount) }
    hipCheck(srtSetDevice(Int32(gpuId)))
    return HipDeviceMemory(deviceIndex, byteCount, stream)
  }

  /// role of CudaQueue.copyAsync (CudaQueue.swift:112-153)
  @inlinable public func copyAsync(from src: DeviceMemory, to dst: DeviceMemory) {
    assert(src.buffer.count == dst.buffer.count)
    let kind: srtMemcpyKind
    switch (src.type, dst.type) {
    case (.unified, .discrete): kind = srtMemcpyHostToDevice
    case (.discrete, .unified): kind = srtMemcpyDeviceToHost
    case (.discrete, .discrete): kind = srtMemcpyDeviceToDevice
    default:
      dst.buffer.copyMemory(from: UnsafeRawBufferPointer(src.buffer))
      return
    }
    hipCheck(srtMemcpyAsync(dst.mutablePointer, src.pointer, src.buffer.count, kind, stream))
  }

  @inlinable public func recordEvent() -> HipEvent {
    let event = HipEvent(options: defaultQueueEventOptions)
    if useGpu { hipCheck(srtEventRecord(event.handle, stream)) }
    return event
  }
  @inlinable public func wait(for event: HipEvent) {
    if useGpu { hipCheck(srtStreamWaitEvent(stream, event.handle)) } else { event.wait() }
  }
  @inlinable public func waitForCompletion() {
    if useGpu { hipCheck(srtStreamSynchronize(stream)) }
  }
}
