/* C ABI of libreactant_mi355x.so: the MI355X (gfx950) execution backend that sits
 * where Reactant.jl calls libReactantExtra's PJRT wrappers.
 *
 * Every entry point below keeps the name, argument order and ownership rules of
 * the reference export it replaces (deps/ReactantExtra/API.cpp, line cited per
 * function), so the Julia side (the files under src/xla/PJRT) can route a call here by
 * swapping the library it `@ccall`s.  Handles are opaque pointers.  The only
 * signature that differs is compilation: the reference passes an in-memory
 * MlirModule; this library takes the module as MLIR text (`string(mod)`).
 *
 * Errors: an entry point that fails records a message (RxLastError), calls the
 * installed `ReactantThrowError` callback if there is one (reference
 * API.cpp:262-270; the Julia callback throws through the C frames), and
 * otherwise returns NULL / 0.  Constructors that take `const char **error`
 * also store a malloc'd message there (API.cpp:568-573).
 *
 * Threading: any thread may call; frees may arrive from finalizer threads at
 * any time (src/xla/PJRT/Buffer.jl:105-111).  Work on one device is ordered on
 * one HIP stream.
 */
#ifndef REACTANT_MI355X_H
#define REACTANT_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct RxClient RxClient;          /* stands for xla::PjRtClient            */
typedef struct RxDevice RxDevice;          /* stands for xla::PjRtDevice            */
typedef struct RxBuffer RxBuffer;          /* stands for xla::PjRtBuffer            */
typedef struct RxExecutable RxExecutable;  /* stands for xla::PjRtLoadedExecutable  */
typedef struct RxFuture RxFuture;          /* stands for xla::Future<>              */

/* API.cpp:262 -- set by the host language at load time. */
extern void (*ReactantThrowError)(const char *);

/* ---- client / device -------------------------------------------------- */
/* API.cpp:528-582 MakeGPUClient.  node_id/num_nodes/distributed client must
 * describe a single process; allowed_devices selects HIP device ordinals
 * (NULL: device 0).  platform_name is accepted and ignored ("rocm"). */
RxClient *MakeGPUClient(int node_id, int num_nodes, int64_t *allowed_devices, int64_t num_allowed_devices,
                        double memory_fraction, bool preallocate, const char *platform_name,
                        const char **error, void *distributed_runtime_client);
void FreeClient(RxClient *client);                                   /* API.cpp:1254 */
int ClientNumDevices(RxClient *client);                              /* API.cpp:688  */
int ClientNumAddressableDevices(RxClient *client);                   /* API.cpp:692  */
int ClientProcessIndex(RxClient *client);                            /* API.cpp:696  */
RxDevice *ClientGetDevice(RxClient *client, int device_id);          /* API.cpp:700  */
RxDevice *ClientGetAddressableDevice(RxClient *client, int device_id); /* API.cpp:704 */
const char *ClientGetPlatformName(RxClient *client);                 /* API.cpp:710, malloc'd */
void ClientGetDevices(RxClient *client, RxDevice **out_devices);     /* API.cpp:718  */
void ClientGetAddressableDevices(RxClient *client, RxDevice **out_devices); /* API.cpp:726 */
const char *DeviceGetKind(RxDevice *device);                         /* API.cpp:714, malloc'd */
RxClient *DeviceToClient(RxDevice *device);                          /* API.cpp:803  */
int64_t PjRtDeviceGetLocalDeviceId(RxDevice *device);                /* API.cpp:1256 */
int64_t PjRtDeviceGetGlobalDeviceId(RxDevice *device);               /* API.cpp:1260 */
int64_t PjRtDeviceGetLocalHardwareId(RxDevice *device);              /* API.cpp:1264 */
bool pjrt_device_is_addressable(RxDevice *device);                   /* API.cpp:3296 */

/* API.cpp:734-765; absent optional fields hold INT64_MIN. */
typedef struct JLAllocatorStats {
  int64_t num_allocs, bytes_in_use, peak_bytes_in_use, largest_alloc_size, bytes_limit, bytes_reserved,
      peak_bytes_reserved, bytes_reservable_limit, largest_free_block_bytes, pool_bytes, peak_pool_bytes;
} JLAllocatorStats;
void PjRtDeviceGetAllocatorStats(RxDevice *device, JLAllocatorStats *stats);

/* ---- buffers ------------------------------------------------------------ */
/* API.cpp:1080-1098.  `ptype` is an xla::PrimitiveType code (src/xla/Utils.jl:18-40),
 * `cshape` the row-major dims (Julia dims reversed, src/xla/PJRT/Buffer.jl:9-17).
 * Host memory is read before the call returns. */
RxBuffer *ArrayFromHostBuffer(RxClient *client, void *data, uint64_t ptype, size_t dim, const int64_t *cshape,
                              RxDevice *device);
/* API.cpp:1230-1241 */
RxBuffer *UninitPJRTBuffer(RxClient *client, RxDevice *device, uint64_t ptype, uint64_t shapeLen, uint64_t *shape);
void BufferToHost(RxBuffer *buffer, void *data);                     /* API.cpp:1162-1177, blocking */
void CopyToBuffer(RxClient *client, RxBuffer *buffer, void *data, size_t offset, size_t size,
                  RxBuffer **bufferP);                               /* API.cpp:1100-1130 */
void CopyFromBuffer(RxClient *client, RxBuffer *buffer, void *data, size_t offset, size_t size,
                    RxBuffer **bufferP);                             /* API.cpp:1179-1197 */
const int64_t *BufferShape(RxBuffer *buffer);                        /* API.cpp:789, borrowed */
int64_t BufferNDimensions(RxBuffer *buffer);                         /* API.cpp:793  */
int BufferPrimitiveType(RxBuffer *buffer);                           /* API.cpp:797  */
RxDevice *BufferToDevice(RxBuffer *buffer);                          /* API.cpp:781  */
RxClient *BufferToClient(RxBuffer *buffer);                          /* API.cpp:785  */
uint8_t BufferOnCPU(RxBuffer *buffer);                               /* API.cpp:1243 */
void *UnsafeBufferPointer(RxBuffer *buffer);                         /* API.cpp:1075 */
RxBuffer *CopyBufferToDevice(RxBuffer *buffer, RxDevice *dst_device);/* API.cpp:1247 */
void PjRtBufferFree(RxBuffer *buffer);                               /* API.cpp:801  */

/* ---- compile / execute ---------------------------------------------------- */
/* Replaces ClientCompileWithProto (API.cpp:1528-1536; Julia side
 * src/xla/PJRT/LoadedExecutable.jl:62-83).  `mlir_text` is the optimized
 * StableHLO module as text; the options proto is accepted and ignored. */
RxExecutable *ClientCompileFromText(RxClient *client, const char *mlir_text, size_t mlir_len,
                                    const char *compile_options_proto, size_t compile_options_proto_size);
void ExecutableFree(RxExecutable *exec);                             /* API.cpp:777  */
RxClient *PjRtLoadedExecutableGetClient(RxExecutable *exec);         /* API.cpp:807  */
/* API.cpp:2064-2071: there are no HLO modules here; *nmodules is set to 0. */
void PjRtLoadedExecutableGetHloModules(RxExecutable *exec, void **hlo_modules, int32_t *nmodules);
/* pjrt_hlo_module_cost_analysis_properties (API.cpp:3238-3260; Julia: XLA.cost_analysis, src/xla/Stats.jl:86-115) takes a
 * HeldHloModule, which this library does not keep.  This entry point fills the same struct of eleven floats
 * (JLHloCostAnalysisProperties: flops, transcendentals, bytes accessed, optimal seconds, utilization, operand 0 / 1
 * utilization, operand 0 / 1 bytes accessed, output root bytes accessed, reserved) for an executable, counted over the
 * StableHLO module it was compiled from. */
void RxExecutableCostAnalysis(RxExecutable *exec, float *properties11);
/* API.cpp:1585-1630.  Results are owning handles; *futures is set to 1 and one
 * future per result is returned.  A donated argument (is_arg_donatable[i] != 0)
 * gives up its storage: the handle stays valid only for PjRtBufferFree. */
void XLAExecuteSharded(RxExecutable *exec, int num_args, RxBuffer **op_args, RxDevice *device,
                       uint8_t *is_arg_donatable, int num_results, RxBuffer **op_results, uint8_t *futures,
                       RxFuture **future_results);
/* A future completes when its device's stream has reached the point at which the future was first asked
 * (FutureIsReady / FutureAwait), which is no earlier than the end of the call that returned it.
 * Calls that wait for the device (these, BufferToHost, CopyFromBuffer) also report a kernel whose bounded wait for
 * another workgroup of its launch expired: they raise once, and the results of that execution are invalid. */
void FreeFuture(RxFuture *future);                                   /* API.cpp:1358 */
uint8_t FutureIsReady(RxFuture *future);                             /* API.cpp:1360 */
void FutureAwait(RxFuture *future);                                  /* API.cpp:1364 */
void InitializeLogs(void);                                           /* API.cpp:414  */
void SetLogLevel(int level);                                         /* API.cpp:430  */

/* ---- additions with no counterpart in the reference ----------------------- */
/* 1 if `handle` was created by this library and is still alive.  Lets patched
 * PJRT wrappers route a Ptr{Cvoid} to this library or to libReactantExtra
 * without dereferencing a foreign pointer. */
int RxOwns(const void *handle);
/* Message of the last failed call on this thread ("" if none); borrowed. */
const char *RxLastError(void);
void RxClearError(void);
/* Parse, plan and compile for gfx950 without a device (build-time check).  Returns 0 on
 * success; *report (malloc'd, may be NULL) receives the fusion plan and, if
 * `with_source` is set, the generated HIP text. */
int RxCompileOffline(const char *mlir_text, size_t mlir_len, int with_source, char **report);
/* Fusion plan of a loaded executable: text report / number of kernel launches /
 * per-launch facts (kernel symbol and kind are borrowed strings). */
const char *RxExecutableReport(RxExecutable *exec);
int RxExecutableNumLaunches(RxExecutable *exec);
int RxExecutableNumResults(RxExecutable *exec);
void RxExecutableLaunchInfo(RxExecutable *exec, int index, const char **kernel, const char **kind,
                            double *algorithmic_bytes, double *flops);
/* XLAExecuteSharded with a HIP event pair attached to every kernel launch (start and stop
 * of the dispatch itself, on the stream the kernels run on); launch_ms has
 * RxExecutableNumLaunches entries. */
void RxExecuteTimed(RxExecutable *exec, int num_args, RxBuffer **op_args, RxDevice *device,
                    uint8_t *is_arg_donatable, int num_results, RxBuffer **op_results, float *launch_ms);
/* The same event pairs without blocking: the call returns as soon as the launches are queued
 * and the events stay with the executable.  RxExecutableTakeTimings waits for the profiled
 * executions queued so far, adds each launch's milliseconds into launch_ms_sum
 * (RxExecutableNumLaunches entries), forgets them and returns how many executions it summed. */
void RxExecuteProfiled(RxExecutable *exec, int num_args, RxBuffer **op_args, RxDevice *device,
                       uint8_t *is_arg_donatable, int num_results, RxBuffer **op_results);
int RxExecutableTakeTimings(RxExecutable *exec, double *launch_ms_sum);
/* No counterpart in the reference.  For callers that cannot allocate device memory while they run
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the launch
 * list of `exec`, like XLAExecuteSharded, but the caller passes the result buffers too (existing
 * buffers of the executable's result types, distinct from the arguments and from each other; they
 * are overwritten), and every temporary of the plan (partial results of the two-pass reductions,
 * tensors handed from one kernel to the next) lives in a static device array of
 * RxNoAllocScratchBytes() = 4 MiB that each GPU the library runs on holds until the process ends.
 * No hipMalloc / hipFree, no event, no handle is created; nothing is donated; the kernels are queued
 * on the device's stream and the call does not wait for them.  Returns 0, or 1 with a message
 * (RxLastError) when the temporaries of the plan exceed the array ("RESOURCE_EXHAUSTED"), or a
 * buffer has the wrong type or device.  All calls on one GPU share the array: calls through one
 * client are ordered by its stream, calls through different clients of the same GPU race. */
int RxExecuteNoAlloc(RxExecutable *exec, int num_args, RxBuffer **op_args, int num_results, RxBuffer **op_results);
size_t RxNoAllocScratchBytes(void);
/* Blocks until all work queued on the device's stream has finished. */
void RxDeviceSynchronize(RxDevice *device);
/* Plain 16-byte-per-lane copy kernel of `bytes` bytes, `iters` times; returns
 * the mean milliseconds per launch (HIP events).  Reference point for HBM
 * bandwidth and for scaling rocprofv3 FETCH_SIZE/WRITE_SIZE readings. */
float RxCalibrationCopy(RxDevice *device, size_t bytes, int iters);
/* Measurement aid, no counterpart in the reference: the rate the MFMA pipe sustains on this device when nothing
 * else runs (one wavefront per SIMD issuing independent MFMAs on register operands for about 10 ms, so that the
 * clock settles under the power limit).  kind 0: v_mfma_f32_16x16x32_bf16, kind 1: v_mfma_f32_16x16x128_f8f6f4 on
 * e4m3; operands pseudo-random, or all zero (`zero_operands` != 0: no toggling in the multipliers).  Writes the
 * TFLOP/s and the average shader clock in MHz; returns 0, or 1 with a message (RxLastError). */
int RxMfmaCeiling(RxDevice *device, int kind, int zero_operands, double *tflops, double *clock_mhz);
/* No counterpart in the reference (measurement aid).  The benchmark's two large GEMM kernels (kind 0: bf16
 * 8192 x 4096 x 4096 on the interleaved streaming body, kind 1: f8E4M3FN 8192^3, kind 2: the bf16 product on the
 * ping-pong body that compiled programs take) launched back to back, timed once the device has been under that load
 * for 150 ms, with a probe inside: out8 = { us per launch, TFLOP/s, cycle counter / real-time counter over the
 * workgroups' lifetimes in MHz, [kinds 0, 1] the same over a sleep of known length that one wavefront of every 16th
 * workgroup takes in the middle of its K loop in MHz (the rest of its workgroup soon waits at a barrier: the clock
 * of an idle compute unit on the loaded chip), cycles counted over that sleep (65024 by the sleep instruction's
 * definition), [kind 2] cycles counted per compute phase (64 MFMAs issued back to back by one wavefront: 1024 at
 * the full rate), cycle counter / real-time counter over those phases in MHz (the clock of a compute unit while
 * its MFMA pipes are full), nanoseconds per compute phase }. */
int RxGemmClockProbe(RxDevice *device, int kind, double *out8);

#ifdef __cplusplus
}
#endif
#endif
