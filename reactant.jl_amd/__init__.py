"""Host side of the MI355X backend, mirroring the part of Reactant.jl that sits
above the runtime C ABI.

Julia is not available where this package is developed, so the host layer that
Reactant implements in `src/xla/PJRT/*.jl` is mirrored here in Python over the
same C entry points (ctypes).  Names and behaviour follow the reference:

    Reactant.set_default_backend("gpu")      src/Reactant.jl:401-404, src/xla/XLA.jl:180-185
    Reactant.to_rarray(x) / ConcreteRArray   src/Tracing.jl:2160-2171, src/Types.jl:214-263
    XLA.PJRT.Client / Device / Buffer        src/xla/PJRT/{Client,Device,Buffer}.jl
    XLA.compile, XLA.execute_sharded         src/xla/PJRT/LoadedExecutable.jl:62-83,175-246
    XLA.PJRT.Future (await / is_ready)       src/xla/PJRT/Future.jl:1-28
    Array(x) (device -> host)                src/ConcreteRArray.jl:108-136
    errors -> ReactantInternalError          src/xla/Utils.jl:3-15

Arrays follow Julia's convention: an array of size (d1, ..., dn) is column-major
on the host and reaches the device as a dense row-major buffer with the dims
REVERSED (src/xla/PJRT/Buffer.jl:9-17).  `to_rarray(x)` therefore uploads
`x.T` (C order) with shape `x.shape[::-1]`; `ConcreteRArray.to_array()` undoes it.

What replaces `@compile f(args...)`: the tracing front end (Julia -> StableHLO)
is not part of this backend; `compile(mlir_text)` takes the optimized module
text that `@compile` would hand to `XLA.compile` and returns the same kind of
callable (`Thunk`, src/compiler/Thunk.jl:9-18,72-86).

The HIP library is required: importing this package without
libreactant_mi355x.so raises, there is no CPU path.
"""
import ctypes
import os

import numpy as np

from . import hostfloat

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libreactant_mi355x.so")


class ReactantInternalError(RuntimeError):
    """Same role as Reactant.XLA.ReactantInternalError (src/xla/Utils.jl:3-15)."""


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libreactant_mi355x.so is not built (run `python reactant.jl_amd/build.py`); "
            "this backend has no fallback path")
    return ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_LOCAL)


lib = _load()

_vp, _i, _i64, _u64, _sz, _cp, _u8 = (ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_uint64,
                                      ctypes.c_size_t, ctypes.c_char_p, ctypes.c_uint8)
_P = ctypes.POINTER


class JLAllocatorStats(ctypes.Structure):
    _fields_ = [(n, _i64) for n in (
        "num_allocs", "bytes_in_use", "peak_bytes_in_use", "largest_alloc_size", "bytes_limit",
        "bytes_reserved", "peak_bytes_reserved", "bytes_reservable_limit", "largest_free_block_bytes",
        "pool_bytes", "peak_pool_bytes")]


# name -> (restype, argtypes); the list is also what the ABI test checks against the header
SIGNATURES = {
    "MakeGPUClient": (_vp, [_i, _i, _P(_i64), _i64, ctypes.c_double, ctypes.c_bool, _cp, _P(_cp), _vp]),
    "FreeClient": (None, [_vp]),
    "ClientNumDevices": (_i, [_vp]),
    "ClientNumAddressableDevices": (_i, [_vp]),
    "ClientProcessIndex": (_i, [_vp]),
    "ClientGetDevice": (_vp, [_vp, _i]),
    "ClientGetAddressableDevice": (_vp, [_vp, _i]),
    "ClientGetPlatformName": (_vp, [_vp]),
    "ClientGetDevices": (None, [_vp, _P(_vp)]),
    "ClientGetAddressableDevices": (None, [_vp, _P(_vp)]),
    "DeviceGetKind": (_vp, [_vp]),
    "DeviceToClient": (_vp, [_vp]),
    "PjRtDeviceGetLocalDeviceId": (_i64, [_vp]),
    "PjRtDeviceGetGlobalDeviceId": (_i64, [_vp]),
    "PjRtDeviceGetLocalHardwareId": (_i64, [_vp]),
    "pjrt_device_is_addressable": (ctypes.c_bool, [_vp]),
    "PjRtDeviceGetAllocatorStats": (None, [_vp, _P(JLAllocatorStats)]),
    "ArrayFromHostBuffer": (_vp, [_vp, _vp, _u64, _sz, _P(_i64), _vp]),
    "UninitPJRTBuffer": (_vp, [_vp, _vp, _u64, _u64, _P(_u64)]),
    "BufferToHost": (None, [_vp, _vp]),
    "CopyToBuffer": (None, [_vp, _vp, _vp, _sz, _sz, _P(_vp)]),
    "CopyFromBuffer": (None, [_vp, _vp, _vp, _sz, _sz, _P(_vp)]),
    "BufferShape": (_P(_i64), [_vp]),
    "BufferNDimensions": (_i64, [_vp]),
    "BufferPrimitiveType": (_i, [_vp]),
    "BufferToDevice": (_vp, [_vp]),
    "BufferToClient": (_vp, [_vp]),
    "BufferOnCPU": (_u8, [_vp]),
    "UnsafeBufferPointer": (_vp, [_vp]),
    "CopyBufferToDevice": (_vp, [_vp, _vp]),
    "PjRtBufferFree": (None, [_vp]),
    "ClientCompileFromText": (_vp, [_vp, _cp, _sz, _cp, _sz]),
    "ExecutableFree": (None, [_vp]),
    "PjRtLoadedExecutableGetClient": (_vp, [_vp]),
    "PjRtLoadedExecutableGetHloModules": (None, [_vp, _P(_vp), _P(ctypes.c_int32)]),
    "XLAExecuteSharded": (None, [_vp, _i, _P(_vp), _vp, _P(_u8), _i, _P(_vp), _P(_u8), _P(_vp)]),
    "FreeFuture": (None, [_vp]),
    "FutureIsReady": (_u8, [_vp]),
    "FutureAwait": (None, [_vp]),
    "InitializeLogs": (None, []),
    "SetLogLevel": (None, [_i]),
    "RxOwns": (_i, [_vp]),
    "RxLastError": (_cp, []),
    "RxClearError": (None, []),
    "RxCompileOffline": (_i, [_cp, _sz, _i, _P(_vp)]),
    "RxExecutableReport": (_cp, [_vp]),
    "RxExecutableNumLaunches": (_i, [_vp]),
    "RxExecutableNumResults": (_i, [_vp]),
    "RxExecutableLaunchInfo": (None, [_vp, _i, _P(_cp), _P(_cp), _P(ctypes.c_double), _P(ctypes.c_double)]),
    "RxExecuteTimed": (None, [_vp, _i, _P(_vp), _vp, _P(_u8), _i, _P(_vp), _P(ctypes.c_float)]),
    "RxExecuteProfiled": (None, [_vp, _i, _P(_vp), _vp, _P(_u8), _i, _P(_vp)]),
    "RxExecutableTakeTimings": (_i, [_vp, _P(ctypes.c_double)]),
    "RxExecuteNoAlloc": (_i, [_vp, _i, _P(_vp), _i, _P(_vp)]),
    "RxNoAllocScratchBytes": (_sz, []),
    "RxDeviceSynchronize": (None, [_vp]),
    "RxCalibrationCopy": (ctypes.c_float, [_vp, _sz, _i]),
    "RxMfmaCeiling": (_i, [_vp, _i, _i, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]),
    "RxGemmClockProbe": (_i, [_vp, _i, ctypes.POINTER(ctypes.c_double)]),
    "RxExecutableCostAnalysis": (None, [_vp, ctypes.POINTER(ctypes.c_float)]),
}
for _name, (_res, _args) in SIGNATURES.items():
    _fn = getattr(lib, _name)
    _fn.restype = _res
    _fn.argtypes = _args

_libc = ctypes.CDLL(None)
_libc.free.argtypes = [_vp]


def _check():
    msg = lib.RxLastError()
    if msg:
        text = msg.decode(errors="replace")
        lib.RxClearError()
        raise ReactantInternalError(text)


def _call(name, *args):
    lib.RxClearError()
    r = getattr(lib, name)(*args)
    _check()
    return r


def _take_string(p):
    """Copy and free a malloc'd C string (reference: unsafe_string_and_free, src/xla/Utils.jl:51-55)."""
    if not p:
        return ""
    s = ctypes.string_at(p).decode()
    _libc.free(p)
    return s


# ----------------------------------------------------------------------------
# element types (xla::PrimitiveType codes, src/xla/Utils.jl:18-40)
# ----------------------------------------------------------------------------
PRIMITIVE_TYPE = {"i1": 1, "i8": 2, "i16": 3, "i32": 4, "i64": 5, "ui8": 6, "ui16": 7, "ui32": 8, "ui64": 9,
                  "f16": 10, "f32": 11, "f64": 12, "bf16": 16, "f8E5M2": 19, "f8E4M3FN": 20}
_NAME_OF_CODE = {v: k for k, v in PRIMITIVE_TYPE.items()}
_STORAGE = {"i1": np.uint8, "i8": np.int8, "i16": np.int16, "i32": np.int32, "i64": np.int64, "ui8": np.uint8,
            "ui16": np.uint16, "ui32": np.uint32, "ui64": np.uint64, "f16": np.float16, "f32": np.float32,
            "f64": np.float64, "bf16": np.uint16, "f8E5M2": np.uint8, "f8E4M3FN": np.uint8}
_NUMPY_DEFAULT = {np.dtype(np.bool_): "i1", np.dtype(np.int8): "i8", np.dtype(np.int16): "i16",
                  np.dtype(np.int32): "i32", np.dtype(np.int64): "i64", np.dtype(np.uint8): "ui8",
                  np.dtype(np.uint16): "ui16", np.dtype(np.uint32): "ui32", np.dtype(np.uint64): "ui64",
                  np.dtype(np.float16): "f16", np.dtype(np.float32): "f32", np.dtype(np.float64): "f64"}


def encode(values, dtype):
    """Numbers -> storage array for `dtype` (rounds to nearest even for narrow floats)."""
    if dtype == "bf16":
        return hostfloat.f32_to_bf16_bits(np.asarray(values, dtype=np.float32)).reshape(np.shape(values))
    if dtype == "f8E4M3FN":
        return hostfloat.f32_to_f8e4m3fn_bits(np.asarray(values, dtype=np.float32)).reshape(np.shape(values))
    if dtype == "f8E5M2":
        return hostfloat.f32_to_f8e5m2_bits(np.asarray(values, dtype=np.float32)).reshape(np.shape(values))
    if dtype == "i1":
        return (np.asarray(values) != 0).astype(np.uint8)
    return np.asarray(values, dtype=_STORAGE[dtype])


def decode(storage, dtype):
    """Storage array -> numbers (float32 for narrow floats, bool for i1)."""
    if dtype == "bf16":
        return hostfloat.bf16_bits_to_f32(storage).reshape(np.shape(storage))
    if dtype == "f8E4M3FN":
        return hostfloat.f8e4m3fn_bits_to_f32(storage)
    if dtype == "f8E5M2":
        return hostfloat.f8e5m2_bits_to_f32(storage)
    if dtype == "i1":
        return np.asarray(storage) != 0
    return np.asarray(storage)


# ----------------------------------------------------------------------------
# XLA.PJRT mirror
# ----------------------------------------------------------------------------
class Device:
    def __init__(self, handle, client):
        self.handle = handle
        self.client = client

    def kind(self):
        return _take_string(_call("DeviceGetKind", self.handle))

    def local_device_id(self):
        return _call("PjRtDeviceGetLocalDeviceId", self.handle)

    def local_hardware_id(self):
        return _call("PjRtDeviceGetLocalHardwareId", self.handle)

    def is_addressable(self):
        return bool(_call("pjrt_device_is_addressable", self.handle))

    def allocator_stats(self):
        st = JLAllocatorStats()
        _call("PjRtDeviceGetAllocatorStats", self.handle, ctypes.byref(st))
        null = -(2 ** 63)
        return {n: (None if getattr(st, n) == null else getattr(st, n)) for n, _ in st._fields_}

    def synchronize(self):
        _call("RxDeviceSynchronize", self.handle)


class Client:
    """XLA.PJRT.Client for platform "rocm" (src/accelerators/GPU.jl:7-37,82-89)."""

    def __init__(self, allowed_devices=None, memory_fraction=0.75, preallocate=False):
        err = _cp()
        arr = None
        n = 0
        if allowed_devices:
            n = len(allowed_devices)
            arr = (_i64 * n)(*allowed_devices)
        lib.RxClearError()
        h = lib.MakeGPUClient(0, 1, arr, n, memory_fraction, preallocate, b"rocm", ctypes.byref(err), None)
        if not h:
            msg = err.value.decode() if err.value else (lib.RxLastError() or b"").decode()
            lib.RxClearError()
            raise ReactantInternalError(msg)
        self.handle = h
        self._devices = None

    def platform_name(self):
        return _take_string(_call("ClientGetPlatformName", self.handle))

    def num_devices(self):
        return _call("ClientNumDevices", self.handle)

    def num_addressable_devices(self):
        return _call("ClientNumAddressableDevices", self.handle)

    def process_index(self):
        return _call("ClientProcessIndex", self.handle)

    def devices(self):
        if self._devices is None:
            n = self.num_devices()
            out = (_vp * n)()
            _call("ClientGetDevices", self.handle, out)
            self._devices = [Device(out[k], self) for k in range(n)]
        return self._devices

    def default_device(self):
        return self.devices()[0]

    def close(self):
        if self.handle:
            for key in [k for k in _THUNKS if k[0] == id(self)]:   # executables of this client go with it
                del _THUNKS[key]
            lib.FreeClient(self.handle)
            self.handle = None


class Future:
    def __init__(self, handle):
        self.handle = handle

    def is_ready(self):
        return bool(_call("FutureIsReady", self.handle))

    def wait(self):
        _call("FutureAwait", self.handle)

    def __del__(self):
        if getattr(self, "handle", None):
            lib.FreeFuture(self.handle)
            self.handle = None


class Buffer:
    """XLA.PJRT.Buffer: owns one device buffer handle (src/xla/PJRT/Buffer.jl)."""

    def __init__(self, handle, client):
        self.handle = handle
        self.client = client

    @staticmethod
    def from_host(client, raw, dtype, device=None):
        """`raw` is the C-ordered storage array in device (reversed-dims) layout."""
        device = device or client.default_device()
        raw = np.asarray(raw, dtype=_STORAGE[dtype])
        if not raw.flags.c_contiguous:
            raw = raw.copy(order="C")  # (np.ascontiguousarray would turn a 0-d array into 1-d)
        dims = (_i64 * raw.ndim)(*raw.shape)
        h = _call("ArrayFromHostBuffer", client.handle, raw.ctypes.data_as(_vp), PRIMITIVE_TYPE[dtype],
                  raw.ndim, dims, device.handle)
        return Buffer(h, client)

    @staticmethod
    def uninitialized(client, shape, dtype, device=None):
        device = device or client.default_device()
        dims = (_u64 * len(shape))(*shape)
        return Buffer(_call("UninitPJRTBuffer", client.handle, device.handle, PRIMITIVE_TYPE[dtype], len(shape),
                            dims), client)

    def shape(self):
        n = _call("BufferNDimensions", self.handle)
        p = _call("BufferShape", self.handle)
        return tuple(p[k] for k in range(n))

    def dtype(self):
        return _NAME_OF_CODE[_call("BufferPrimitiveType", self.handle)]

    def on_cpu(self):
        return bool(_call("BufferOnCPU", self.handle))

    def unsafe_pointer(self):
        return _call("UnsafeBufferPointer", self.handle)

    def to_host(self):
        """Storage array in device layout (blocking)."""
        dt = self.dtype()
        out = np.empty(self.shape(), dtype=_STORAGE[dt])
        _call("BufferToHost", self.handle, out.ctypes.data_as(_vp))
        return out

    def copy_to_host(self, out, offset_bytes=0):
        _call("CopyFromBuffer", self.client.handle, self.handle, out.ctypes.data_as(_vp), offset_bytes, out.nbytes,
              None)

    def copy_from_host(self, src, offset_bytes=0):
        src = np.ascontiguousarray(src)
        _call("CopyToBuffer", self.client.handle, self.handle, src.ctypes.data_as(_vp), offset_bytes, src.nbytes,
              None)

    def copy(self):
        dev = _call("BufferToDevice", self.handle)
        return Buffer(_call("CopyBufferToDevice", self.handle, dev), self.client)

    def free(self):
        if self.handle:
            lib.PjRtBufferFree(self.handle)
            self.handle = None

    def __del__(self):
        self.free()


class AsyncBuffer:
    """Buffer plus the future of the execution that produces it (src/xla/PJRT/AsyncBuffer.jl:1-4)."""

    def __init__(self, buffer, future=None):
        self.buffer = buffer
        self.future = future

    def synced_buffer(self):
        if self.future is not None:
            self.future.wait()
            self.future = None
        return self.buffer


class LoadedExecutable:
    """XLA.PJRT.LoadedExecutable (src/xla/PJRT/LoadedExecutable.jl)."""

    def __init__(self, handle, client):
        self.handle = handle
        self.client = client
        self.num_results = _call("RxExecutableNumResults", handle)

    def report(self):
        return _call("RxExecutableReport", self.handle).decode()

    def launches(self):
        out = []
        for k in range(_call("RxExecutableNumLaunches", self.handle)):
            kn, kd, b, f = _cp(), _cp(), ctypes.c_double(), ctypes.c_double()
            _call("RxExecutableLaunchInfo", self.handle, k, ctypes.byref(kn), ctypes.byref(kd), ctypes.byref(b),
                  ctypes.byref(f))
            out.append({"kernel": kn.value.decode(), "kind": kd.value.decode(), "algorithmic_bytes": b.value,
                        "flops": f.value})
        return out

    def cost_analysis(self):
        """XLA.cost_analysis(exec) (src/xla/Stats.jl:86-115): the fields of HloCostAnalysisProperties as a dict."""
        props = (ctypes.c_float * 11)()
        _call("RxExecutableCostAnalysis", self.handle, props)
        names = ("flops", "transcendentals", "bytes_accessed", "optimal_seconds", "utilization", "operand0_utilization",
                 "operand1_utilization", "operand0_bytes_accessed", "operand1_bytes_accessed", "output_root_bytes_accessed", "reserved0")
        return dict(zip(names, [float(v) for v in props]))

    def get_hlo_modules(self):
        n = ctypes.c_int32(-1)
        _call("PjRtLoadedExecutableGetHloModules", self.handle, None, ctypes.byref(n))
        return [None] * n.value

    def execute_sharded(self, buffers, donated=None, device=None):
        """XLA.execute_sharded: returns AsyncBuffers (src/xla/PJRT/LoadedExecutable.jl:175-246)."""
        n = len(buffers)
        args = (_vp * n)(*[b.handle for b in buffers])
        don = (_u8 * n)(*([1 if d else 0 for d in donated] if donated else [0] * n))
        nres = self.num_results
        res = (_vp * nres)()
        futs = (_vp * nres)()
        has = _u8(0)
        dev = (device or self.client.default_device()).handle
        _call("XLAExecuteSharded", self.handle, n, args, dev, don, nres, res, ctypes.byref(has), futs)
        out = []
        for k in range(nres):
            out.append(AsyncBuffer(Buffer(res[k], self.client), Future(futs[k]) if has.value else None))
        return out

    def execute_timed(self, buffers, donated=None, device=None):
        """Like execute_sharded, with a HIP event pair around every kernel launch: (buffers, ms list)."""
        n = len(buffers)
        args = (_vp * n)(*[b.handle for b in buffers])
        don = (_u8 * n)(*([1 if d else 0 for d in donated] if donated else [0] * n))
        nres = self.num_results
        res = (_vp * nres)()
        nl = _call("RxExecutableNumLaunches", self.handle)
        ms = (ctypes.c_float * max(nl, 1))()
        dev = (device or self.client.default_device()).handle
        _call("RxExecuteTimed", self.handle, n, args, dev, don, nres, res, ms)
        return [Buffer(res[k], self.client) for k in range(nres)], [ms[k] for k in range(nl)]

    def execute_profiled(self, buffers, donated=None, device=None):
        """Like execute_timed but does not wait: the event pairs are read later by take_timings()."""
        n = len(buffers)
        args = (_vp * n)(*[b.handle for b in buffers])
        don = (_u8 * n)(*([1 if d else 0 for d in donated] if donated else [0] * n))
        nres = self.num_results
        res = (_vp * nres)()
        dev = (device or self.client.default_device()).handle
        _call("RxExecuteProfiled", self.handle, n, args, dev, don, nres, res)
        return [Buffer(res[k], self.client) for k in range(nres)]

    def execute_no_alloc(self, buffers, results):
        """Queue the launch list with caller-owned result buffers and every temporary in the library's
        static device array (4 MiB): nothing is allocated, nothing is donated, no future is returned."""
        n, nres = len(buffers), len(results)
        args = (_vp * n)(*[b.handle for b in buffers])
        res = (_vp * nres)(*[b.handle for b in results])
        _call("RxExecuteNoAlloc", self.handle, n, args, nres, res)

    def take_timings(self):
        """(number of profiled executions since the last call, per-launch mean milliseconds)."""
        nl = _call("RxExecutableNumLaunches", self.handle)
        acc = (ctypes.c_double * max(nl, 1))()
        runs = _call("RxExecutableTakeTimings", self.handle, acc)
        return runs, [acc[k] / max(runs, 1) for k in range(nl)]

    def free(self):
        if self.handle:
            lib.ExecutableFree(self.handle)
            self.handle = None

    def __del__(self):
        self.free()


def xla_compile(client, mlir_text):
    """XLA.compile(client, mod): module text in, LoadedExecutable out."""
    data = mlir_text.encode() if isinstance(mlir_text, str) else bytes(mlir_text)
    h = _call("ClientCompileFromText", client.handle, data, len(data), None, 0)
    return LoadedExecutable(h, client)


def mfma_ceiling(device, kind, zero_operands=False):
    """(TFLOP/s, average shader clock in MHz) the MFMA pipe sustains on `device` with nothing else running:
    kind "bf16" (v_mfma_f32_16x16x32_bf16) or "f8" (v_mfma_f32_16x16x128_f8f6f4), pseudo-random or all-zero operands."""
    tf, mhz = ctypes.c_double(), ctypes.c_double()
    _call("RxMfmaCeiling", device.handle, {"bf16": 0, "f8": 1}[kind], 1 if zero_operands else 0, ctypes.byref(tf), ctypes.byref(mhz))
    return tf.value, mhz.value


def gemm_clock_probe(device, kind):
    """The benchmark's large GEMM kernel of `kind` ("bf16": 8192 x 4096 x 4096 on the interleaved streaming body, "f8":
    8192^3, "bf16_pingpong": the bf16 product on the ping-pong body that compiled programs take) launched back to back, timed
    once the device has been under that load for 150 ms, with a probe inside: dict with us per launch, TFLOP/s, the ratio of
    the shader-cycle counter to the real-time counter over the workgroups' lifetimes (MHz); for "bf16" and "f8" the same
    ratio over a sleep of known length that one wavefront takes in the middle of the K loop (MHz: its workgroup soon waits at
    a barrier, so this is the clock of an idle compute unit on the loaded chip) and the cycles counted over that sleep (65024
    nominal); for "bf16_pingpong" the cycles counted per compute phase (64 MFMAs issued back to back: 1024 at the full rate),
    the same ratio over those phases (MHz: the clock of a compute unit while its MFMA pipes are full) and ns per phase."""
    out = (ctypes.c_double * 8)()
    _call("RxGemmClockProbe", device.handle, {"bf16": 0, "f8": 1, "bf16_pingpong": 2}[kind], out)
    res = {"us_per_launch": out[0], "TFLOP/s": out[1], "lifetime_cycles_over_real_time_MHz": out[2]}
    if kind == "bf16_pingpong":
        res.update({"cycles_per_compute_phase_of_64_MFMAs": out[5], "compute_phase_cycles_over_real_time_MHz": out[6], "ns_per_compute_phase": out[7]})
    else:
        res.update({"clock_MHz": out[3], "cycles_over_a_sleep_of_65024": out[4]})
    return res


def compile_offline(mlir_text, with_source=False):
    """Parse, plan and compile for gfx950 without a device; returns the plan report."""
    data = mlir_text.encode()
    rep = _vp()
    rc = lib.RxCompileOffline(data, len(data), 1 if with_source else 0, ctypes.byref(rep))
    text = _take_string(rep.value)
    lib.RxClearError()
    if rc != 0:
        raise ReactantInternalError(text)
    return text


# ----------------------------------------------------------------------------
# top-level API
# ----------------------------------------------------------------------------
_state = {"client": None, "backend": None}


def set_default_backend(name):
    """Reactant.set_default_backend: "gpu" and "rocm" select this backend; anything else is an error
    (the CPU/TPU clients of the reference are other runtimes, not part of this library)."""
    if name not in ("gpu", "rocm"):
        raise ReactantInternalError('backend "%s" is not provided by the MI355X runtime (use "gpu")' % name)
    if _state["client"] is None:
        _state["client"] = Client()
    _state["backend"] = name
    return _state["client"]


def default_backend():
    if _state["client"] is None:
        set_default_backend("gpu")
    return _state["client"]


class ConcreteRArray:
    """ConcretePJRTArray{T,N}: shape in Julia order + one AsyncBuffer (src/Types.jl:214-227)."""

    def __init__(self, data, shape, dtype):
        self.data = data          # AsyncBuffer
        self.shape = tuple(shape)  # Julia order
        self.dtype = dtype
        self.donated = False

    def _buffer(self):
        if self.donated:
            raise ReactantInternalError("accessing the data of a donated array")  # src/Types.jl:9-26
        return self.data.synced_buffer()

    def to_array(self):
        """Array(x): numbers in Julia index order (float32 for narrow floats)."""
        raw = self._buffer().to_host()
        return decode(raw, self.dtype).T

    def to_storage(self):
        return self._buffer().to_host().T

    def __array__(self, dtype=None):
        a = self.to_array()
        return a.astype(dtype) if dtype is not None else a

    # -- array operations that go through the device (src/ConcreteRArray.jl:423-446,783-805,
    #    src/xla/PJRT/Buffer.jl:19-103,170-182).  Indices are 1-based, as in Julia. ------------
    def _client(self):
        return self.data.buffer.client

    def _tensor_type(self):
        return "tensor<" + "".join("%dx" % d for d in self.shape[::-1]) + self.dtype + ">"

    def similar(self, dtype=None, shape=None):
        """Base.similar: an uninitialized array on the same device."""
        dtype, shape = dtype or self.dtype, tuple(shape if shape is not None else self.shape)
        buf = Buffer.uninitialized(self._client(), shape[::-1], dtype)
        return ConcreteRArray(AsyncBuffer(buf), shape, dtype)

    def copy(self):
        return ConcreteRArray(AsyncBuffer(self._buffer().copy()), self.shape, self.dtype)

    def _swap(self, thunk, *extra):
        """Run an updating function with this array donated and take over the result's buffer
        (in-place updates are handle swaps: src/compiler/Codegen.jl:1151-1169)."""
        out = thunk(self, *extra, donated=[True] + [False] * len(extra))
        self.data, self.donated = out.data, False
        return self

    def fill(self, value):
        """fill!(a, value): compiles `broadcast_in_dim` of a number and runs it."""
        if 0 in self.shape:
            raise ReactantInternalError("Cannot setindex! to empty buffer")
        tt, st = self._tensor_type(), "tensor<%s>" % self.dtype
        text = ("module @reactant_fill {\n  func.func @main(%%arg0: %s {tf.aliasing_output = 0 : i32}, %%arg1: %s) -> %s {\n"
                "    %%0 = stablehlo.broadcast_in_dim %%arg1, dims = [] : (%s) -> %s\n    return %%0 : %s\n  }\n}\n"
                % (tt, st, tt, st, tt, tt))
        return self._swap(_cached_thunk(self._client(), text), to_rarray(np.asarray(value), self.dtype, self._client()))

    def _index_module(self, store):
        n = len(self.shape)
        tt, st, it = self._tensor_type(), "tensor<%s>" % self.dtype, "tensor<i64>"
        one = "tensor<" + "1x" * n + self.dtype + ">"
        first = 2 if store else 1                                       # position of the first index argument
        idx_args = "".join(", %%arg%d: %s" % (k + first, it) for k in range(n))
        body = "    %c = stablehlo.constant dense<1> : tensor<i64>\n"
        for k in range(n):
            body += "    %%i%d = stablehlo.subtract %%arg%d, %%c : %s\n" % (k, k + first, it)
        starts = ", ".join("%%i%d" % k for k in reversed(range(n)))     # dims are reversed on the device
        its = ", ".join([it] * n)
        if store:
            body += "    %%u = stablehlo.reshape %%arg1 : (%s) -> %s\n" % (st, one)
            body += "    %%r = stablehlo.dynamic_update_slice %%arg0, %%u, %s : (%s, %s, %s) -> %s\n" % (starts, tt, one, its, tt)
            return ("module @reactant_mysetindex {\n  func.func @main(%%arg0: %s {tf.aliasing_output = 0 : i32}, %%arg1: %s%s) -> %s {\n%s"
                    "    return %%r : %s\n  }\n}\n" % (tt, st, idx_args, tt, body, tt))
        body += "    %%s = stablehlo.dynamic_slice %%arg0, %s, sizes = [%s] : (%s, %s) -> %s\n" % (starts, ", ".join(["1"] * n), tt, its, one)
        body += "    %%r = stablehlo.reshape %%s : (%s) -> %s\n" % (one, st)
        return ("module @reactant_mygetindex {\n  func.func @main(%%arg0: %s%s) -> %s {\n%s    return %%r : %s\n  }\n}\n"
                % (tt, idx_args, st, body, st))

    def _check_index(self, idx):
        if len(idx) != len(self.shape) or not self.shape:
            raise IndexError("expected %d indices" % len(self.shape))
        for i, d in zip(idx, self.shape):
            if not 1 <= int(i) <= d:
                raise IndexError("index %r out of bounds for an array of size %r" % (tuple(idx), self.shape))

    def setindex(self, value, *idx):
        """a[i, j, ...] = value for one element (scalar indexing of a device array): compiles a
        `dynamic_update_slice` whose start indices are arguments, so one executable serves
        every position."""
        self._check_index(idx)
        cl = self._client()
        nums = [to_rarray(np.asarray(value), self.dtype, cl)] + [to_rarray(np.int64(i), "i64", cl) for i in idx]
        return self._swap(_cached_thunk(cl, self._index_module(True)), *nums)

    def getindex(self, *idx):
        """a[i, j, ...] for one element."""
        self._check_index(idx)
        cl = self._client()
        nums = [to_rarray(np.int64(i), "i64", cl) for i in idx]
        out = _cached_thunk(cl, self._index_module(False))(self, *nums)
        return out.to_array()[()]


def to_rarray(x, dtype=None, client=None):
    """Reactant.to_rarray: host array (Julia index order) -> device."""
    client = client or default_backend()
    x = np.asarray(x)
    if dtype is None:
        dtype = _NUMPY_DEFAULT[x.dtype]
    storage = encode(x, dtype)
    raw = storage.T.copy(order="C")
    return ConcreteRArray(AsyncBuffer(Buffer.from_host(client, raw, dtype)), x.shape, dtype)


class Thunk:
    """Callable produced by compile (reference: src/compiler/Thunk.jl:9-18,72-86)."""

    def __init__(self, exec_, client):
        self.exec = exec_
        self.client = client

    def __call__(self, *args, donated=None, sync=False):
        bufs = [a._buffer() for a in args]
        res = self.exec.execute_sharded(bufs, donated)
        if donated:
            for a, d in zip(args, donated):
                if d:
                    a.donated = True
        outs = []
        for ab in res:
            if sync:
                ab.synced_buffer()
            b = ab.buffer
            outs.append(ConcreteRArray(ab, b.shape()[::-1], b.dtype()))
        return outs[0] if len(outs) == 1 else tuple(outs)


def compile(mlir_text, client=None):
    client = client or default_backend()
    return Thunk(xla_compile(client, mlir_text), client)


_THUNKS = {}


def _cached_thunk(client, mlir_text):
    """One executable per (client, module text): the small functions behind fill!/setindex!/getindex."""
    key = (id(client), mlir_text)
    if key not in _THUNKS:
        _THUNKS[key] = compile(mlir_text, client)
    return _THUNKS[key]


# ----------------------------------------------------------------------------
# Reactant.Serialization.export_to_enzymejax hand-off (src/serialization/EnzymeJAX.jl:124-172)
# ----------------------------------------------------------------------------
def load_enzymejax_export(mlir_path, npz_path=None):
    """Read what `export_to_enzymejax` writes for one function: `<fn>_<id>.mlir` (the module as
    `string(mod)`) and `<fn>_<id>_inputs.npz` with keys `arr_1 … arr_N` in `@main` argument order.
    The arrays were saved with their dims reversed (`permutedims(arr, reverse(1:ndims(arr)))`,
    ext/ReactantNPZExt.jl:9-22), i.e. already in the layout of the module's tensor types; numbers
    are 0-d.  Returns (module text, [numpy arrays])."""
    with open(mlir_path, "r") as f:
        text = f.read()
    if npz_path is None:
        stem = mlir_path[:-5] if mlir_path.endswith(".mlir") else mlir_path
        npz_path = stem + "_inputs.npz"
    arrays = []
    with np.load(npz_path, allow_pickle=False) as z:
        keys = set(z.files)
        k = 1
        while "arr_%d" % k in keys:
            arrays.append(np.asarray(z["arr_%d" % k]))
            k += 1
        if len(arrays) != len(keys):
            raise ReactantInternalError("%s: expected keys arr_1 … arr_N, found %s" % (npz_path, sorted(keys)))
    return text, arrays


def run_enzymejax_export(mlir_path, npz_path=None, client=None):
    """Compile an exported module, upload its saved inputs and run it once.  Returns the results
    as numpy arrays in the module's (dim-reversed) layout — what the generated Python script's
    `run_<fn>(*load_inputs())` returns (src/serialization/EnzymeJAX.jl:338-345,390-402); the
    Julia-order array is `result.T` for every rank."""
    client = client or default_backend()
    text, arrays = load_enzymejax_export(mlir_path, npz_path)
    exe = xla_compile(client, text)
    bufs = []
    for i, a in enumerate(arrays):
        if a.dtype not in _NUMPY_DEFAULT:
            raise ReactantInternalError("input arr_%d has dtype %s, which no tensor element type stores" % (i + 1, a.dtype))
        dt = _NUMPY_DEFAULT[a.dtype]
        bufs.append(Buffer.from_host(client, encode(a, dt), dt))
    outs = exe.execute_sharded(bufs)
    res = []
    for ab in outs:
        b = ab.synced_buffer()
        res.append(decode(b.to_host(), b.dtype()))
    return res
