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
// CudaEvent}.swift and are written requirement by requirement against the protocols in
// platform/common/Platform.swift:37-71, :280-330 and platform/common/DeviceQueue.swift:22-82
// (`Logging` and `deviceName` have default implementations there: common/Log.swift:200-207,
// DeviceQueue.swift:129-133).  They import the C module of include/srt_hip.h.
//
// UNCOMPILED: this environment has no Swift toolchain.  The sources have been checked against
// the protocol declarations by reading, not by a compiler.
//******************************************************************************
import Foundation
import SwiftRTHip

//==============================================================================
/// hipCheck: role of cudaCheck(cudaError_t) (CudaPlatform.swift:180-193).  Any status other
/// than success is a hard error: log on the current queue and trap.
@inlinable public func hipCheck(
  _ status: srtStatus,
  file: String = #file,
  function: String = #function,
  line: Int = #line
) {
  if status != srtSuccess {
    let location = "HIP error in \(file) at \(function):\(line)"
    let message = String(cString: srtGetStatusString(status))
    _ = srtDeviceSynchronize()
    currentQueue.writeLog("\(message) at \(location)")
    fatalError("unrecoverable error")
  }
}

/// hipCheck(stream): role of cudaCheck(cudaStream_t) (CudaPlatform.swift:160-177).  In DEBUG builds
/// every launch is followed by a stream synchronization so that asynchronous errors surface at the
/// call that caused them (the native module built with `make DEBUG=1` does the same on its side).
@inlinable public func hipCheck(
  _ stream: srtStream?,
  file: String = #file,
  function: String = #function,
  line: Int = #line
) {
  #if DEBUG
    hipCheck(srtStreamSynchronize(stream), file: file, function: function, line: line)
  #endif
}

//==============================================================================
/// HipPlatform: role of CudaPlatform (CudaPlatform.swift:22-115)
public class HipPlatform: ComputePlatform {
  // types
  public typealias Storage = DiscreteStorage

  // shared (the static requirements of ComputePlatform, Platform.swift:44-70)
  public static var cpuQueueCount = 0
  public static let discreteMemoryDeviceId = 1
  public static let eventId = AtomicCounter()
  public static let local = HipPlatform()
  public static let mainThread = pthread_self()
  public static let objectId = AtomicCounter()
  public static let queueId = AtomicCounter()
  public static let startTime = Date()
  public static var lastRandomSeed: RandomSeed = generateRandomSeed()

  public static var acceleratorQueueCount: Int = 2 {
    didSet {
      precondition(acceleratorQueueCount > 0, "there must be at least 1 accelerator queue")
    }
  }

  /// for synchronous execution and syncing with the app thread (cpu, no stream)
  public static let syncQueue =
    HipQueue(deviceIndex: 0, name: "appThread", queueMode: .sync, useGpu: false)

  // instance state
  public var devices: [HipDevice]
  public let logInfo: LogInfo
  public let name: String
  public var queueStack: [HipQueue]

  /// the shared single-zero storage AD uses for Element.zero (CudaPlatform.swift:60-66)
  public static let zeroStorage: Storage = {
    Storage(storedElement: Int64(0), name: "Zero")
  }()

  @inlinable public init() {
    // device 0 is the cpu, as in the reference's numbering; HipDevice covers both kinds so that no
    // existential is needed
    let cpuDevice = HipDevice(index: 0)
    devices = [cpuDevice]
    if devices[0].queues.count == 0 {
      devices[0].queues.append(Self.syncQueue)
    }

    queueStack = []
    var gpuDeviceCount: Int32 = 0
    hipCheck(srtGetDeviceCount(&gpuDeviceCount))
    for i in 1..<Int(gpuDeviceCount + 1) {
      devices.append(HipDevice(index: i))
    }

    name = "\(Self.self)"
    logInfo = LogInfo(logWriter: log, logLevel: .error, namePath: name, nestingLevel: 0)

    // the first gpu's queue 0 is the default
    if gpuDeviceCount > 0 {
      queueStack = [devices[1].queues[0]]
    } else {
      queueStack = [Self.syncQueue]
      writeLog("There are no '\(self.name)' devices installed", level: .warning)
    }
    diagnostic(.device, "default: \(queueStack[0].name)", categories: .device)
  }
}

//==============================================================================
/// cpuFallback: role of CudaPlatform.swift:117-144.  srtErrorNotSupported means the native module
/// declined the layout or element type: run the same op on the cpu device's queue instead.
@usableFromInline func _cpuFallback(_ body: (Platform.Device.Queue) -> Void) {
  let name = currentQueue.deviceName
  using(device: 0) {
    currentQueue.diagnostic(
      .fallback, "unsupported function on \(name) delegated to \(currentQueue.name)",
      categories: .fallback)
    body(currentQueue)
  }
}

@inlinable public func cpuFallback(_ status: srtStatus, _ body: (Platform.Device.Queue) -> Void) {
  if status == srtErrorNotSupported {
    _cpuFallback(body)
  } else {
    hipCheck(status)
  }
}

//==============================================================================
/// HipDevice: role of CudaDevice (CudaDevice.swift:22-94)
public final class HipDevice: ComputeDevice {
  public let index: Int
  public let memoryType: MemoryType
  public let name: String
  public var queues: [HipQueue]

  @inlinable public init(index: Int) {
    let isCpu = index == 0
    self.index = index
    self.name = "dev:\(index)"
    self.memoryType = isCpu ? .unified : .discrete
    queues = []

    let description = isCpu ? getCpuProperties() : getHipDeviceProperties()
    diagnostic(.device, "\(name) \(description)", categories: .device)

    if isCpu {
      for i in 0..<Platform.cpuQueueCount {
        queues.append(
          HipQueue(deviceIndex: index, name: "\(name)_q\(i)", queueMode: .async, useGpu: false))
      }
    } else {
      for i in 0..<Platform.acceleratorQueueCount {
        queues.append(
          HipQueue(deviceIndex: index, name: "\(name)_q\(i)", queueMode: .async, useGpu: true))
      }
    }
  }

  /// device 0 is the cpu, so the gpu hardware index is one less
  @inlinable public func select() { hipCheck(srtSetDevice(Int32(index - 1))) }

  @inlinable func getCpuProperties() -> String {
    let info = ProcessInfo.processInfo
    let oneGB = UInt64(1) << 30
    return "[type: cpu, cores: \(info.activeProcessorCount), memory: "
      + "\(info.physicalMemory / oneGB + 1) GB, addressing: \(memoryType)]"
  }

  @inlinable func getHipDeviceProperties() -> String {
    var props = srtDeviceProperties()
    hipCheck(srtGetDeviceProperties(&props, Int32(index - 1)))
    let deviceName = withUnsafePointer(to: &props.name) {
      $0.withMemoryRebound(to: UInt8.self, capacity: MemoryLayout.size(ofValue: props.name)) {
        String(cString: $0)
      }
    }
    return "[type: \(deviceName), multiprocessors: \(props.multiProcessorCount), "
      + "memory: \(props.totalGlobalMem >> 30) GB, addressing: \(memoryType)]"
  }
}

//==============================================================================
/// HipDeviceMemory: role of CudaDeviceMemory (CudaDevice.swift:96-162).  The Swift object owns
/// the pointer; the native module keeps no reference to tensor memory.
public final class HipDeviceMemory: DeviceMemory {
  public let buffer: UnsafeMutableRawBufferPointer
  public let deviceIndex: Int
  public var name: String?
  public var releaseMessage: String?
  public let type: MemoryType
  public var version: Int
  public let isReference: Bool
  /// the stream the block was allocated on: the allocator reuses it there at once
  public let stream: srtStream?

  @inlinable public var mutablePointer: UnsafeMutableRawPointer {
    UnsafeMutableRawPointer(buffer.baseAddress!)
  }
  @inlinable public var pointer: UnsafeRawPointer {
    UnsafeRawPointer(buffer.baseAddress!)
  }

  @inlinable public init(_ deviceIndex: Int, _ byteCount: Int, _ stream: srtStream?) {
    self.deviceIndex = deviceIndex
    self.stream = stream
    // pad to the widest vector access (32 bytes, as CudaDevice.swift:141-142 does with double4)
    let paddedByteCount = roundUp(byteCount, multiple: 32)
    var devicePointer: UnsafeMutableRawPointer?
    hipCheck(srtDeviceAllocate(&devicePointer, paddedByteCount, stream))
    self.buffer = UnsafeMutableRawBufferPointer(start: devicePointer!, count: byteCount)
    self.type = .discrete
    self.isReference = false
    self.version = -1
    self.releaseMessage = nil
  }

  /// The free is ordered on the allocating stream.  Storage that was last written or read on another
  /// queue has already made this queue wait for that work (DiscreteStorage.swift:271-296 synchronizes
  /// replicas across queues with events before a buffer changes hands).
  @inlinable deinit {
    hipCheck(srtDeviceFree(buffer.baseAddress!))
    #if DEBUG
      if let name = name, let msg = releaseMessage {
        diagnostic(.release, "\(name)\(msg)", categories: .dataAlloc)
      }
    #endif
  }
}

//==============================================================================
/// HipEvent: role of CudaEvent (CudaEvent.swift:23-75)
public class HipEvent: QueueEvent, Logging {
  public let id = Platform.eventId.next
  // used to synchronize with a cpu async queue
  @usableFromInline let cpuEvent: DispatchSemaphore
  // used to synchronize with a stream
  @usableFromInline let handle: srtEvent

  @inlinable public init(recordedOn queue: HipQueue, options: QueueEventOptions = []) {
    // blocking only for the async cpu case; signaled for sync cpu and streams so wait() falls through
    let value = queue.deviceIndex == 0 && queue.mode == .async ? 0 : 1
    cpuEvent = DispatchSemaphore(value: value)
    var temp: srtEvent?
    hipCheck(srtEventCreate(&temp, options.contains(.timing) ? 1 : 0))
    handle = temp!
  }

  @inlinable deinit {
    _ = srtEventDestroy(handle)
  }

  /// only called by the cpu async queue implementation
  @inlinable public func signal() {
    cpuEvent.signal()
    _ = srtEventRecord(handle, nil)
  }

  @inlinable public func wait() {
    // wait for the first occurrence, then let all other waiters through
    cpuEvent.wait()
    cpuEvent.signal()
    _ = srtEventSynchronize(handle)
  }

  @inlinable public var occurred: Bool { srtEventQuery(handle) == srtSuccess }
}

//==============================================================================
/// HipQueue: role of CudaQueue (CudaQueue.swift:22-196): one non-blocking stream on one device.
/// The functions it overrides live in HipMatmul.swift and HipMath.swift; everything else comes
/// from CpuFunctions' defaults.
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
  /// DeviceQueue.deviceName (a default exists, DeviceQueue.swift:129-133; spelled out for the record)
  @inlinable public var deviceName: String { platform.devices[deviceIndex].name }

  @inlinable public init(
    deviceIndex: Int,
    name: String,
    queueMode: DeviceQueueMode,
    useGpu: Bool
  ) {
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
      var hipStream: srtStream?
      hipCheck(srtStreamCreate(&hipStream))   // non-blocking, default priority
      stream = hipStream
    } else {
      stream = nil   // a cpu queue never reaches the native module (the reference creates a stream here too)
    }
    diagnostic(.create, "queue: \(name)", categories: .queueAlloc)
  }

  @inlinable public func selectDevice() {
    hipCheck(srtSetDevice(Int32(gpuId)))
  }

  /// allocate a device memory buffer suitably aligned for any type
  @inlinable public func allocate(byteCount: Int, heapIndex: Int = 0) -> DeviceMemory {
    if usesCpu {
      let buffer = UnsafeMutableRawBufferPointer.allocate(
        byteCount: byteCount, alignment: MemoryLayout<Int>.alignment)
      return CpuDeviceMemory(deviceIndex, buffer, memoryType)
    } else {
      selectDevice()
      return HipDeviceMemory(deviceIndex, byteCount, stream)
    }
  }

  @inlinable public func delay(_ interval: TimeInterval) {
    guard useGpu else {
      cpu_delay(interval)
      return
    }
    hipCheck(srtDelayStream(interval, stream))
  }

  /// role of CudaQueue.copyAsync (CudaQueue.swift:112-153)
  @inlinable public func copyAsync(from src: DeviceMemory, to dst: DeviceMemory) {
    assert(src.buffer.count == dst.buffer.count)
    switch (src.type, dst.type) {
    case (.unified, .unified):
      cpu_copyAsync(from: src, to: dst)
    case (.unified, .discrete):
      hipCheck(srtMemcpyAsync(dst.mutablePointer, src.pointer, src.buffer.count, srtMemcpyHostToDevice, stream))
    case (.discrete, .unified):
      hipCheck(srtMemcpyAsync(dst.mutablePointer, src.pointer, src.buffer.count, srtMemcpyDeviceToHost, stream))
    case (.discrete, .discrete):
      hipCheck(srtMemcpyAsync(dst.mutablePointer, src.pointer, src.buffer.count, srtMemcpyDeviceToDevice, stream))
    }
  }

  @inlinable public func recordEvent() -> HipEvent {
    let event = HipEvent(recordedOn: self, options: defaultQueueEventOptions)
    if useGpu {
      hipCheck(srtEventRecord(event.handle, stream))
    } else if mode == .async {
      queue.async(group: group) { event.signal() }
    }
    return event
  }

  /// causes this queue to wait until the event has occurred
  @inlinable public func wait(for event: HipEvent) {
    if useGpu {
      hipCheck(srtStreamWaitEvent(stream, event.handle))
    } else if mode == .sync {
      event.wait()
    } else {
      queue.async(group: group) { event.wait() }
    }
  }

  /// the synchronous queue completes work as it is queued, so it is always complete
  @inlinable public func waitForCompletion() {
    if useGpu {
      hipCheck(srtStreamSynchronize(stream))
    } else if mode == .async {
      group.wait()
    }
  }
}
