/*
 * srt_hip.h -- C ABI of the SwiftRTHip native module (MI355X / gfx950).
 *
 * This module fills, for the matmul / Dense path, the role that Sources/CCUDA (the clang
 * module exposing the CUDA runtime) and Modules/SwiftRTCuda (the extern "C" srt* functions)
 * fill in the reference.  A Swift `HipQueue` imports this header through a module map and
 * calls it exactly where `CudaQueue` calls the CUDA runtime and the srt* functions.
 *
 * Conventions (same as the reference's native module):
 *   - every function returns a status; srtSuccess == 0.
 *   - srtErrorNotSupported means "caller, run your CPU fallback"
 *     (role of cudaErrorNotSupported in cpuFallback,
 *     Sources/SwiftRTCore/platform/cuda/device/CudaPlatform.swift:122-144).
 *     Any other non-zero status is a hard error (the reference's cudaCheck resets the device
 *     and traps, CudaPlatform.swift:180-193).
 *   - the native side never throws, aborts or logs; it never retains tensor memory or
 *     descriptor memory after a call returns (descriptors live on the caller's stack,
 *     CudaExtensions.swift:24-84), and kernels are launched asynchronously on `stream`.
 *   - data pointers are already offset to the first element of the view
 *     (Tensor.deviceRead, Sources/SwiftRTCore/tensor/Tensor.swift:558-582); extents and
 *     strides are 64-bit counts of elements.
 *   - plain C types only: no C++ and no framework types cross this boundary.
 */
#pragma once
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* every declaration below is exported from the shared library (it is built with hidden
 * default visibility) */
#pragma GCC visibility push(default)

/* Enumerations cross the boundary as 32-bit integers.  A caller may hand in a value that is none of the
 * enumerators (another cudaDataType id, a tiled order): the library answers srtErrorNotSupported or
 * srtErrorInvalidValue.  In C++ the types get a fixed underlying type so that holding such a value is
 * well defined; in C an enumeration is an integer anyway. */
#ifdef __cplusplus
#define SRT_ENUM(tag) enum tag : int32_t
#else
#define SRT_ENUM(tag) enum tag
#endif

/* ---- status ---------------------------------------------------------------------------- */
typedef int32_t srtStatus;
enum {
  srtSuccess = 0,
  srtErrorInvalidValue = 1,      /* null pointer, rank/extent mismatch, bad enum value        */
  srtErrorOutOfMemory = 2,       /* device or pinned-host allocation failed                   */
  srtErrorNotReady = 600,        /* srtEventQuery: work not finished (not an error)           */
  srtErrorNotSupported = 801,    /* run the CPU fallback (same value as cudaErrorNotSupported) */
  srtErrorLaunchFailure = 719,   /* a launch or an asynchronous error was reported by HIP     */
  srtErrorNoDevice = 100,        /* no gfx950 device visible / HIP runtime failed to start    */
  srtErrorUnknown = 999
};

/* Human-readable name of a status; never NULL; storage is static. */
const char* srtGetStatusString(srtStatus status);

/* ---- element types ----------------------------------------------------------------------
 * Replaces srtDataType, Modules/SwiftRTCuda/tensor_api.h:28-65.  The values the path uses keep
 * the reference's numeric ids (they are the cudaDataType values) so `E.type` in
 * StorageElement.swift:123-129 ports unchanged. */
typedef SRT_ENUM(srtDataType_e) {
  srtUnknownType = -1,
  srtReal32F = 0,
  srtReal64F = 1,   /* declared for completeness; matmul returns srtErrorNotSupported */
  srtReal16F = 2,
  srtReal16BF = 14
} srtDataType;

/* Storage order.  Replaces the cublasLtOrder_t field of srtTensorDescriptor
 * (tensor_api.h:76); same numeric values as CUBLASLT_ORDER_COL / CUBLASLT_ORDER_ROW, which is
 * what `order.cublas` yields (CudaPlatform.swift:297-311).  Strides are authoritative; order
 * is checked only to reject tiled layouts (anything else -> srtErrorNotSupported). */
typedef SRT_ENUM(srtOrder_e) { srtOrderCol = 0, srtOrderRow = 1 } srtOrder;

/* Tensor descriptor.  Replaces srtTensorDescriptor, tensor_api.h:70-87, field for field, so
 * Tensor.withTensor (CudaExtensions.swift:24-84) builds it the same way.  shape / strides /
 * logicalStrides point at `rank` values on the caller's stack; they are read during the call
 * only. */
typedef struct {
  srtDataType type;             /* element type                                              */
  uint32_t rank;                /* number of dimensions                                      */
  srtOrder order;               /* storage order                                             */
  size_t count;                 /* number of logical elements                                */
  size_t spanCount;             /* number of storage elements spanned                        */
  const size_t* shape;          /* extent of each dimension                                  */
  const size_t* strides;        /* storage stride of each dimension, in elements             */
  const size_t* logicalStrides; /* dense logical strides (unused by matmul, may be NULL)     */
} srtTensorDescriptor;

/* Epilogue activation.  Case order and values follow ActivationType,
 * Sources/SwiftRTCore/platform/common/FunctionProperties.swift:44-51 (rawValue ports 1:1). */
typedef SRT_ENUM(srtActivation_e) {
  srtActivationSigmoid = 0,     /* 1 / (1 + exp(-x))                                         */
  srtActivationRelu = 1,        /* max(x, 0)                                                 */
  srtActivationTanh = 2,
  srtActivationClippedRelu = 3, /* min(max(x, 0), coef)   coef = activationReluCeiling       */
  srtActivationElu = 4,         /* x > 0 ? x : coef * (exp(x) - 1)                           */
  srtActivationIdentity = 5
} srtActivation;

/* Opaque handles.  A stream is a HIP stream; an event a HIP event. */
typedef struct srtStream_st* srtStream;
typedef struct srtEvent_st* srtEvent;

/* ---- device ------------------------------------------------------------------------------ */
/* Replaces cudaGetDeviceCount (CudaPlatform.swift:89). */
srtStatus srtGetDeviceCount(int32_t* count);
/* Replaces cudaSetDevice (CudaQueue.swift:62,78; CudaDevice.swift:70). */
srtStatus srtSetDevice(int32_t device);
srtStatus srtGetDevice(int32_t* device);

typedef struct {
  char name[256];
  char archName[64];           /* e.g. "gfx950:sramecc+:xnack-"                               */
  size_t totalGlobalMem;       /* bytes                                                       */
  int32_t multiProcessorCount; /* compute units                                               */
  int32_t clockRateKHz;        /* peak engine clock                                           */
  int32_t memoryClockRateKHz;
  int32_t memoryBusWidthBits;
  int32_t l2CacheBytes;
  int32_t sharedMemPerBlockBytes; /* LDS available to one workgroup                           */
  int32_t warpSize;            /* 64                                                          */
} srtDeviceProperties;
/* Replaces cudaGetDeviceProperties (CudaDevice.swift:88). */
srtStatus srtGetDeviceProperties(srtDeviceProperties* props, int32_t device);
/* Blocks until every stream of the current device is idle (cudaDeviceSynchronize role). */
srtStatus srtDeviceSynchronize(void);

/* ---- streams ----------------------------------------------------------------------------- */
/* Replaces cudaStreamCreateWithFlags(.., cudaStreamNonBlocking) (CudaQueue.swift:65-68).
 * Streams are created at default priority on the current device. */
srtStatus srtStreamCreate(srtStream* stream);
srtStatus srtStreamDestroy(srtStream stream);
/* Replaces cudaStreamSynchronize (CudaQueue.swift:193). */
srtStatus srtStreamSynchronize(srtStream stream);

/* ---- events ------------------------------------------------------------------------------ */
/* Replaces cudaEventCreateWithFlags (CudaEvent.swift:48-50).  enableTiming != 0 makes the
 * event usable with srtEventElapsedTime. */
srtStatus srtEventCreate(srtEvent* event, int32_t enableTiming);
/* Replaces cudaEventDestroy (CudaEvent.swift:55). */
srtStatus srtEventDestroy(srtEvent event);
/* Replaces cudaEventRecord (CudaQueue.swift:159). */
srtStatus srtEventRecord(srtEvent event, srtStream stream);
/* Replaces cudaStreamWaitEvent (CudaQueue.swift:175). */
srtStatus srtStreamWaitEvent(srtStream stream, srtEvent event);
/* Replaces cudaEventSynchronize (CudaEvent.swift:62,70). */
srtStatus srtEventSynchronize(srtEvent event);
/* srtSuccess when complete, srtErrorNotReady otherwise (cudaEventQuery role). */
srtStatus srtEventQuery(srtEvent event);
srtStatus srtEventElapsedTime(float* milliseconds, srtEvent start, srtEvent stop);

/* ---- memory ------------------------------------------------------------------------------ */
/* Replace srtDeviceAllocate / srtDeviceFree, Modules/SwiftRTCuda/memory_api.h:26-27 (called
 * from CudaDeviceMemory, CudaDevice.swift:147,159).  Stream-ordered caching allocator: a
 * freed block is reused at once on the stream it was last used on, and on other streams once
 * the work queued on that stream at the time of the free has finished.  "The stream it was used
 * on" is the stream given to srtDeviceAllocate: a caller that also used the block on another
 * stream orders that work before the free itself (event + srtStreamWaitEvent, as the storage layer
 * does for cross-queue reads, DiscreteStorage.swift:271-296).  Thread safe.  The caller owns the
 * pointer; the library keeps no reference to tensor memory. */
srtStatus srtDeviceAllocate(void** devPtr, size_t size, srtStream stream);
srtStatus srtDeviceFree(void* devPtr);
/* Returns every cached (free) block of every device to the driver. */
srtStatus srtDeviceEmptyCache(void);
/* Pinned host staging memory (newly allocated, never registered in place). */
srtStatus srtHostAllocate(void** hostPtr, size_t size);
srtStatus srtHostFree(void* hostPtr);

typedef SRT_ENUM(srtMemcpyKind_e) {
  srtMemcpyHostToDevice = 1,
  srtMemcpyDeviceToHost = 2,
  srtMemcpyDeviceToDevice = 3
} srtMemcpyKind;
/* Replaces cudaMemcpyAsync (CudaQueue.swift:125-151): ordered on `stream`; host buffers may
 * be pageable. */
srtStatus srtMemcpyAsync(void* dst, const void* src, size_t byteCount, srtMemcpyKind kind,
                         srtStream stream);
/* Fills byteCount bytes with `value` on `stream` using a fill kernel (safe to capture). */
srtStatus srtMemsetAsync(void* dst, int32_t value, size_t byteCount, srtStream stream);

/* ---- matmul ------------------------------------------------------------------------------
 * out = op(a) . op(b), op = optional swap of the last two dimensions (`Tensor.t`,
 * Sources/SwiftRTCore/tensor/TensorInit.swift:844-890).  Rank 2, or rank 3 with a leading
 * batch dimension (batch stride taken from strides[0]; 0 broadcasts an operand).
 *
 * This is the entry point HipQueue.matmul calls, for both overloads, in place of the
 * cpuFallback in CudaQueue.matmul (Sources/SwiftRTCore/platform/cuda/functions/
 * CudaMatmul.swift:25-42 and :44-61); the arithmetic it replaces is cpu_matmul
 * (Sources/SwiftRTCore/platform/cpu/functions/CpuMath.swift:1141-1161, :1164-1186).
 * Elements: srtReal32F, srtReal16F, srtReal16BF, all three tensors the same type.  Products
 * are accumulated in fp32 and rounded once (nearest even) to the element type.
 * Operands may be any strided view; `out` may have any strides, but must share no element with `a`, `b`
 * or the bias (tiles are stored while other tiles are still being read).  Views whose storage spans
 * (first to last element) do not overlap are accepted, and so are overlapping spans that a common pitch
 * proves apart: column slices of one wide row-major buffer, interleaved batches.  `out` starting on an
 * input's first element, or overlapping an input as row blocks of one pitch, is srtErrorInvalidValue; spans that overlap in a way the check cannot resolve are
 * srtErrorNotSupported (the caller's fallback runs).
 *
 * Returns srtErrorNotSupported (caller falls back to the CPU) for other element types,
 * orders other than row/col, or rank other than 2/3; srtErrorInvalidValue when extents do not
 * agree; srtSuccess with no launch when any extent is zero. */
srtStatus srtMatmul(const void* a, const srtTensorDescriptor* aDesc, int32_t transposeA,
                    const void* b, const srtTensorDescriptor* bDesc, int32_t transposeB,
                    void* out, const srtTensorDescriptor* oDesc, srtStream stream);

/* out = activation(op(a) . op(b) + bias), bias broadcast over rows, bias and activation applied
 * to the fp32 accumulators in registers before the single rounding to the element type.
 * This is the Dense forward: it implements what matmul(_:transposed:_:transposed:bias:)
 * (Sources/SwiftRTCore/operators/Matmul.swift:57-72, which drops its bias) and
 * Dense.callAsFunction (Sources/SwiftRTLayers/Dense.swift:36-39, a stub) are meant to compute,
 * and what the recurrent cells compute today as three ops
 * (Sources/SwiftRTLayers/Recurrent.swift:157-161, :255-266).
 * bias: rank-1 tensor of N elements of the same type (bias == NULL: no bias add).
 * coef: ceiling for srtActivationClippedRelu, alpha for srtActivationElu, ignored otherwise.
 * Rank 2 or 3 as srtMatmul (the same bias is applied to every batch). */
srtStatus srtMatmulBiasActivation(const void* a, const srtTensorDescriptor* aDesc, int32_t transposeA,
                                  const void* b, const srtTensorDescriptor* bDesc, int32_t transposeB,
                                  const void* bias, const srtTensorDescriptor* biasDesc,
                                  srtActivation activation, double coef,
                                  void* out, const srtTensorDescriptor* oDesc, srtStream stream);

/* Name of the kernel family the dispatcher selects for this problem ("mfma_256x256_m16_k64", "mfma_256x256_m16_k64_tail",
 * "mfma_128x128_m16_k128", "mfma_128x256_m16_k64", "mfma_256x128_m16_k64", "mfma_256x256_m16", "mfma_256x256", "skinny", "generic", ...; the full
 * list is with srtMatmulTune), written into `name`; nothing is launched.  A 16-bit problem
 * whose operands span 1 Gi elements or more runs as several launches over halves of its batch, M or N;
 * the name is then that of the first piece's kernel followed by "/pieces".  Diagnostic only
 * (the reference's matmul diagnostic line, CudaMatmul.swift:34-37, has no counterpart for
 * kernel choice). */
srtStatus srtMatmulQueryKernel(const srtTensorDescriptor* aDesc, int32_t transposeA,
                               const srtTensorDescriptor* bDesc, int32_t transposeB,
                               const srtTensorDescriptor* oDesc, const void* a, const void* b,
                               const void* out, char* name, size_t nameCapacity);

/* ---- plan / tune cache ------------------------------------------------------------------------
 * The role of ExecutionPlanCache / ExecutionPlanner (Sources/SwiftRTCore/platform/common/
 * ExecutionPlanner.swift:20-29), of the `plan` key a layer keeps (Sources/SwiftRTLayers/Dense.swift:29)
 * and of CudaMatmul2.tune (Sources/SwiftRTCore/platform/cuda/functions/CudaMatmul.swift:112-120, an
 * empty body in the reference).
 *
 * srtMatmulTune takes the arguments of srtMatmulBiasActivation, runs the problem with every kernel
 * plan it qualifies for (a few timed launches each, on `stream`; the call synchronises with the
 * stream), records the fastest in a process-wide cache and leaves `out` computed by it.  The key is
 * the element type, M, N, K, batch, the layout class of the operands (which dimension is contiguous,
 * whether rows keep 16-byte alignment) and the epilogue (bias present, activation).  Every later
 * srtMatmul / srtMatmulBiasActivation call with the same key runs the recorded plan -- provided this
 * call's pointers still meet the plan's alignment rules; otherwise, and for keys never tuned, the
 * built-in heuristic decides.  All plans compute the same function to the documented tolerance
 * (sums are fp32; their order differs between plans).
 * chosen (optional): receives the plan's name ("mfma_256x256_m16_k64", "mfma_256x256_m16_k64_tail" (the same kernel
 * with the tiles left over after its whole rounds cut along k; its result does not depend on timing either),
 * "mfma_256x256_m16_k64_split" (the same kernel with its last round in 192-wide tiles: only ever a tuned or loaded plan),
 * "mfma_128x256_m16_k64" and "mfma_256x128_m16_k64" (the same kernel body on half tiles, for grids that would leave compute
 * units idle in 256 x 256 tiles: 128 rows when A is contiguous along k, 128 columns when it is not),
 * "mfma_128x128_m16_k128" (128 x 128 tiles on 128-deep staging units, any layout, K a multiple of 128 and at least 256: what
 * problems of up to one tile per compute unit run on),
 * "mfma_256x256_m16", "mfma_256x256", "mfma_256x256_k64",
 * "mfma_256x256_splitk", "mfma_128x256_m16", "mfma_128x128", "mfma_64x64", "mfma_128x128_any", "mfma_64x64_any" (16-bit
 * operands of any stride and alignment), "skinny" (16-bit types up to 64 rows, fp32 up to 32), "f32_mfma_128x128_ring", "f32_mfma_64x128_ring", "f32_mfma_64x64_ring" (one
 * fp32 kernel in three tile shapes: K a multiple of 64 and at least 128, operands contiguous along k or along m / n with
 * 16-byte aligned rows), "f32_mfma_128x128_parts" (its k range cut in parts, for a single matrix of a few tiles and a long k),
 * "f32_mfma_64x64", "f32_mfma_splitk", "generic").
 * The cache is thread-safe.  Save / Load use a small text file, one plan per line:
 *   dtype M N K batch layout epilogue plan-name
 * (layout: bit 0 A contiguous along k, 1 A along m, 2 B along k, 3 B along n, 4 result rows
 * contiguous, 5 bias per row of the computed tile, 6 rows 16-byte aligned; epilogue: bit 0 bias
 * present, bits 1.. the srtActivation code), so a tuned set of shapes can be shipped with an
 * application; Load merges into the cache and is
 * all-or-nothing: a malformed file returns srtErrorInvalidValue and changes nothing. */
srtStatus srtMatmulTune(const void* a, const srtTensorDescriptor* aDesc, int32_t transposeA,
                        const void* b, const srtTensorDescriptor* bDesc, int32_t transposeB,
                        const void* bias, const srtTensorDescriptor* biasDesc,
                        srtActivation activation, double coef,
                        void* out, const srtTensorDescriptor* oDesc, srtStream stream,
                        char* chosen, size_t chosenCapacity);
srtStatus srtPlanCacheClear(void);
srtStatus srtPlanCacheCount(size_t* count);
srtStatus srtPlanCacheSave(const char* path);
srtStatus srtPlanCacheLoad(const char* path);

/* ---- backward of the Dense epilogue ------------------------------------------------------------
 * dx = dy * activation'(y) and, when dbias != NULL, dbias[n] = sum over rows of dx[:, n], in one
 * pass over y and dy.  y is the OUTPUT of the forward activation: the derivative is written in
 * terms of it (sigmoid y(1-y), tanh 1-y^2, relu y>0, clippedRelu 0<y<coef, elu y>0 ? 1 : y+coef,
 * identity 1), so the pre-activation need not be kept.
 *
 * Fills the role of CudaActivation.backward (cudnnActivationBackward(y, dy, x) -> dx,
 * Sources/SwiftRTCore/platform/cuda/layers/CudaActivation.swift:101-127) and supplies the bias
 * term of the pullbacks the reference leaves as fatalError() (_vjpMatmul...bias,
 * Sources/SwiftRTCore/differentiable/MathDerivatives.swift:520-554).  The remaining two products of
 * the backward pass are srtMatmul calls with transpose flags (matmulGradients,
 * MathDerivatives.swift:460-482).
 * y, dy, dx: rank 2, [M, N], one element type (32F, 16F, 16BF), any strides; dbias: rank 1, N
 * elements.  Sums are fp32 in a fixed order (results do not vary from run to run).
 * With dbias, takes a stream-ordered workspace of at most max(8 MiB, 4 N bytes) from the library's
 * allocator for the duration of the call's kernels.  srtErrorNotSupported for other ranks or element types. */
srtStatus srtActivationBackwardBias(const void* y, const srtTensorDescriptor* yDesc,
                                    const void* dy, const srtTensorDescriptor* dyDesc,
                                    srtActivation activation, double coef,
                                    void* dx, const srtTensorDescriptor* dxDesc,
                                    void* dbias, const srtTensorDescriptor* dbiasDesc, srtStream stream);

/* The same computation for callers that cannot allocate (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Identical arguments and
 * results (bit for bit) to srtActivationBackwardBias, but the fp32 partial rows of the bias gradient
 * live in a fixed 8 MiB device array inside the library (one per GPU, held until the process ends)
 * instead of a block from the allocator: the call performs no device or host allocation and frees
 * nothing.  Limit: with a bias gradient, N <= 2 097 152 columns (one fp32 partial row must fit the 8 MiB);
 * srtErrorInvalidValue beyond that.  Every call on a GPU shares that GPU's array:
 * calls that overlap in time on one GPU (different streams, or different threads) race; serialise them.
 * The array needs no clearing between calls (every entry read is written first by the same call).
 * The array used is that of the device `stream` belongs to (the current device for the null stream).  Its
 * address is looked up once per device: by srtStreamCreate for the device current at that time, otherwise by
 * the first call on that device -- a lookup is a runtime query, not a launch, so with a stream made elsewhere
 * make one call per device before capturing calls into a graph. */
srtStatus srtActivationBackwardBiasNoAlloc(const void* y, const srtTensorDescriptor* yDesc,
                                           const void* dy, const srtTensorDescriptor* dyDesc,
                                           srtActivation activation, double coef,
                                           void* dx, const srtTensorDescriptor* dxDesc,
                                           void* dbias, const srtTensorDescriptor* dbiasDesc, srtStream stream);

/* ---- element-wise neighbours of the path ---------------------------------------------------------
 * Same names, argument order and conventions as the reference's native module
 * (Modules/SwiftRTCuda/math_api.h: srtAdd :75-100, srtDiv :138-148, srtExp :166-170, srtMul
 * :222-233, srtNeg :268-272, srtSigmoid :285-289, srtSub :315-332, srtTanh :338-342;
 * compare_api.h: srtMin :139-165, srtMax :170-181; copy_api.h: srtCopy :27-38; fill_api.h:
 * srtFillFlat :27-33), called from CudaQueue exactly as there
 * (Sources/SwiftRTCore/platform/cuda/functions/CudaMath.swift:93-150).
 *
 * Strided forms: all tensors the same rank and shape; an input broadcasts along a dimension by
 * giving it stride 0 there (Tensor(repeating:to:)); `out` may be any non-aliasing strided view.
 * TE forms: `element` points to ONE host-side element of the tensors' type, read during the call.
 * Flat forms: dense buffers of `count` elements -- what CudaQueue calls when canFlatten holds
 * (CudaMath.swift:103-113); every binary operator has a tensor-tensor (Flat) and a tensor-element
 * (TEFlat) form.
 * Element types 32F, 16F, 16BF (srtCopy / srtCopyFlat also convert between any two of them,
 * rounding to nearest even); arithmetic is fp32 with one rounding to the element type, i.e. the
 * reference's CPU definitions evaluated in E.Value (CpuMath.swift:646-662, :1189-1256,
 * :1369-1377; max is `a >= b ? a : b`, min `a <= b ? a : b`).
 * Any other element type, or a layout that does not collapse to 4 dimensions: srtErrorNotSupported
 * (caller falls back to the CPU, the reference's convention for unsupported combinations,
 * Modules/SwiftRTCuda/op2.h:276-289). */
srtStatus srtAdd(const void* a, const srtTensorDescriptor* aDesc, const void* b, const srtTensorDescriptor* bDesc,
                 void* out, const srtTensorDescriptor* oDesc, srtStream stream);
srtStatus srtAddTE(const void* a, const srtTensorDescriptor* aDesc, const void* element,
                   void* out, const srtTensorDescriptor* oDesc, srtStream stream);
srtStatus srtAddFlat(srtDataType type, const void* a, const void* b, void* out, size_t count, srtStream stream);
/* Tensor-element on a dense buffer: replaces srtAddTEFlat (math_api.h:95-100), argument order as there. */
srtStatus srtAddTEFlat(const void* a, srtDataType atype, const void* element, void* out, size_t count,
                       srtStream stream);
srtStatus srtSub(const void* a, const srtTensorDescriptor* aDesc, const void* b, const srtTensorDescriptor* bDesc,
                 void* out, const srtTensorDescriptor* oDesc, srtStream stream);
srtStatus srtSubTE(const void* a, const srtTensorDescriptor* aDesc, const void* element,
                   void* out, const srtTensorDescriptor* oDesc, srtStream stream);
srtStatus srtSubFlat(srtDataType type, const void* a, const void* b, void* out, size_t count, srtStream stream);
srtStatus srtSubTEFlat(const void* a, srtDataType atype, const void* element, void* out, size_t count,
                       srtStream stream);
srtStatus srtMul(const void* a, const srtTensorDescriptor* aDesc, const void* b, const srtTensorDescriptor* bDesc,
                 void* out, const srtTensorDescriptor* oDesc, srtStream stream);
srtStatus srtMulTE(const void* a, const srtTensorDescriptor* aDesc, const void* element,
                   void* out, const srtTensorDescriptor* oDesc, srtStream stream);
srtStatus srtMulFlat(srtDataType type, const void* a, const void* b, void* out, size_t count, srtStream stream);
srtStatus srtMulTEFlat(const void* a, srtDataType atype, const void* element, void* out, size_t count,
                       srtStream stream);
srtStatus srtDiv(const void* a, const srtTensorDescriptor* aDesc, const void* b, const srtTensorDescriptor* bDesc,
                 void* out, const srtTensorDescriptor* oDesc, srtStream stream);
srtStatus srtDivTE(const void* a, const srtTensorDescriptor* aDesc, const void* element,
                   void* out, const srtTensorDescriptor* oDesc, srtStream stream);
srtStatus srtDivFlat(srtDataType type, const void* a, const void* b, void* out, size_t count, srtStream stream);
srtStatus srtDivTEFlat(const void* a, srtDataType atype, const void* element, void* out, size_t count,
                       srtStream stream);
srtStatus srtMax(const void* a, const srtTensorDescriptor* aDesc, const void* b, const srtTensorDescriptor* bDesc,
                 void* out, const srtTensorDescriptor* oDesc, srtStream stream);
srtStatus srtMaxTE(const void* a, const srtTensorDescriptor* aDesc, const void* element,
                   void* out, const srtTensorDescriptor* oDesc, srtStream stream);
srtStatus srtMaxFlat(srtDataType type, const void* a, const void* b, void* out, size_t count, srtStream stream);
srtStatus srtMaxTEFlat(const void* a, srtDataType atype, const void* element, void* out, size_t count,
                       srtStream stream);
srtStatus srtMin(const void* a, const srtTensorDescriptor* aDesc, const void* b, const srtTensorDescriptor* bDesc,
                 void* out, const srtTensorDescriptor* oDesc, srtStream stream);
srtStatus srtMinTE(const void* a, const srtTensorDescriptor* aDesc, const void* element,
                   void* out, const srtTensorDescriptor* oDesc, srtStream stream);
srtStatus srtMinFlat(srtDataType type, const void* a, const void* b, void* out, size_t count, srtStream stream);
srtStatus srtMinTEFlat(const void* a, srtDataType atype, const void* element, void* out, size_t count,
                       srtStream stream);
/* The reference's comparison family spells its dense tensor-element form with the type first
 * (srtMinFlatTE, compare_api.h:160-167); both spellings are exported for max and min. */
srtStatus srtMinFlatTE(srtDataType type, const void* a, const void* element, void* out, size_t count, srtStream stream);
srtStatus srtMaxFlatTE(srtDataType type, const void* a, const void* element, void* out, size_t count, srtStream stream);
srtStatus srtNeg(const void* a, const srtTensorDescriptor* aDesc,
                 void* out, const srtTensorDescriptor* oDesc, srtStream stream);
srtStatus srtExp(const void* a, const srtTensorDescriptor* aDesc,
                 void* out, const srtTensorDescriptor* oDesc, srtStream stream);
srtStatus srtSigmoid(const void* a, const srtTensorDescriptor* aDesc,
                     void* out, const srtTensorDescriptor* oDesc, srtStream stream);
srtStatus srtTanh(const void* a, const srtTensorDescriptor* aDesc,
                  void* out, const srtTensorDescriptor* oDesc, srtStream stream);
srtStatus srtCopy(const void* a, const srtTensorDescriptor* aDesc,
                  void* out, const srtTensorDescriptor* oDesc, srtStream stream);
srtStatus srtCopyFlat(srtDataType atype, const void* a, srtDataType otype, void* out, size_t count,
                      srtStream stream);
srtStatus srtFillFlat(srtDataType type, void* out, const void* element, size_t count, srtStream stream);

/* ---- test helper ------------------------------------------------------------------------- */
/* Replaces srtDelayStream, Modules/SwiftRTCuda/utilities_api.h:28: occupies `stream` for about
 * `seconds` (bounded spin on the device clock; at most 10 s). */
srtStatus srtDelayStream(double seconds, srtStream stream);

/* Library version: major * 10000 + minor * 100 + patch. */
int32_t srtGetVersion(void);

#pragma GCC visibility pop

#ifdef __cplusplus
}
#endif
