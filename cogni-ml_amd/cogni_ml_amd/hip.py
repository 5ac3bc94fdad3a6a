"""ML::HIP: Python (ctypes) binding of the driver layer in libcogni_hip.so.

Mirrors the reference's ML::CUDA module (src/ml/cuda/driver.cr:53-343) class for class:
Context, DeviceBuffer, HIPModule (CUDAModule), KernelFunction, FunctionAttribute, HIPStream,
HIPGraph, HIPGraphExec, with_stream, copy_htod/dtoh/dtod, synchronize, launch and
ResidentSequenceRunner, with the same ownership rules (one handle per wrapper, idempotent
close, no finalizers) and the same error rule (non-zero status raises, driver.cr:57-59).
"""
import contextlib
import ctypes
import enum
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_PKG), "lib", "libcogni_hip.so")

_lib = None


class HIPError(RuntimeError):
    def __init__(self, what, code):
        self.code = code
        name = lib().mlhip_error_string(code).decode() if code > 0 else ""
        super().__init__("%s failed with HIP error %d%s" % (what, code, " (%s)" % name if name else ""))


def lib():
    """Load libcogni_hip.so. There is no fallback: a missing library is an error."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: build it with `make -C cogni-ml_amd/csrc` "
                               "(or __graft_entry__.build())" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        L.mlhip_error_string.restype = ctypes.c_char_p
        L.mlhip_error_string.argtypes = [ctypes.c_int]
        L.cogni_last_error.restype = ctypes.c_char_p
        L.cogni_gemv_kernel_name.restype = ctypes.c_char_p
        L.cogni_gemv_kernel_name.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_int]
        L.cogni_dequantize_kernel_name.restype = ctypes.c_char_p
        L.cogni_dequantize_kernel_name.argtypes = [ctypes.c_uint32]
        L.cogni_data_bytes.restype = ctypes.c_int64
        L.cogni_data_bytes.argtypes = [ctypes.c_uint32, ctypes.c_int64]
        L.cogni_weight_device_ptr.restype = ctypes.c_uint64
        L.cogni_weight_device_ptr.argtypes = [ctypes.c_void_p]
        L.mlhip_mem_alloc.argtypes = [ctypes.POINTER(ctypes.c_uint64), ctypes.c_size_t]
        L.mlhip_mem_free.argtypes = [ctypes.c_uint64]
        L.mlhip_memcpy_htod.argtypes = [ctypes.c_uint64, ctypes.c_void_p, ctypes.c_size_t]
        L.mlhip_memcpy_dtoh.argtypes = [ctypes.c_void_p, ctypes.c_uint64, ctypes.c_size_t]
        L.mlhip_memcpy_dtod.argtypes = [ctypes.c_uint64, ctypes.c_uint64, ctypes.c_size_t]
        L.mlhip_module_load_data.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p]
        L.mlhip_module_unload.argtypes = [ctypes.c_void_p]
        L.mlhip_module_get_function.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p, ctypes.c_char_p]
        L.mlhip_func_get_attribute.argtypes = [ctypes.POINTER(ctypes.c_int32), ctypes.c_int32, ctypes.c_void_p]
        L.mlhip_stream_create.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_uint32]
        for f in ("mlhip_stream_destroy", "mlhip_stream_synchronize", "mlhip_graph_destroy",
                  "mlhip_graph_exec_destroy", "mlhip_event_synchronize", "mlhip_event_destroy", "mlhip_ctx_destroy"):
            getattr(L, f).argtypes = [ctypes.c_void_p]
        L.mlhip_stream_begin_capture.argtypes = [ctypes.c_void_p, ctypes.c_int32]
        L.mlhip_stream_end_capture.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p)]
        L.mlhip_graph_instantiate.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p, ctypes.c_uint64]
        L.mlhip_graph_upload.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        L.cogni_gemv_release_stream.argtypes = [ctypes.c_void_p]
        L.mlhip_graph_launch.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        L.mlhip_launch_kernel.argtypes = [ctypes.c_void_p] + [ctypes.c_uint32] * 7 + [
            ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p]
        L.mlhip_event_create.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        L.mlhip_event_record.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        L.mlhip_event_elapsed_ms.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        L.mlhip_ctx_create.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_uint32, ctypes.c_int32]
        _lib = L
    return _lib


_current_stream = None  # module-global, like @@current_stream (driver.cr:55)


def check(code, what):
    """ML::CUDA.check! (driver.cr:57-59)."""
    if code != 0:
        raise HIPError(what, code)


class Context:
    """driver.cr:61-94."""

    def __init__(self, handle, device, device_name, cc_major, cc_minor, arch, compute_units, clock_khz):
        self._handle, self.device = handle, device
        self.device_name, self.arch = device_name, arch
        self.compute_capability_major, self.compute_capability_minor = cc_major, cc_minor
        self.compute_units, self.clock_khz = compute_units, clock_khz
        self._closed = False

    @classmethod
    def create(cls, ordinal=0):
        L = lib()
        check(L.mlhip_init(0), "hipInit")
        dev = ctypes.c_int32()
        check(L.mlhip_device_get(ctypes.byref(dev), ordinal), "hipDeviceGet")
        buf = ctypes.create_string_buffer(256)
        check(L.mlhip_device_get_name(buf, 256, dev), "hipDeviceGetName")
        name = buf.value.decode().strip()
        major, minor = ctypes.c_int32(), ctypes.c_int32()
        check(L.mlhip_device_compute_capability(ctypes.byref(major), ctypes.byref(minor), dev),
              "hipDeviceComputeCapability")
        check(L.mlhip_device_get_arch(buf, 256, dev), "hipGetDeviceProperties")
        arch = buf.value.decode()
        cu, clk = ctypes.c_int32(), ctypes.c_int32()
        check(L.mlhip_device_get_cu_clock(ctypes.byref(cu), ctypes.byref(clk), dev), "hipDeviceGetAttribute")
        handle = ctypes.c_void_p()
        check(L.mlhip_ctx_create(ctypes.byref(handle), 0, dev), "hipCtxCreate")
        return cls(handle, dev.value, name, major.value, minor.value, arch, cu.value, clk.value)

    def close(self):
        if self._closed:
            return
        lib().mlhip_ctx_destroy(self._handle)
        self._closed = True


class DeviceBuffer:
    """driver.cr:96-112: owns one device allocation."""

    def __init__(self, bytesize):
        self.bytesize = int(bytesize)
        p = ctypes.c_uint64(0)
        check(lib().mlhip_mem_alloc(ctypes.byref(p), max(self.bytesize, 1)), "hipMalloc")
        self.ptr = p.value
        self._closed = False

    def close(self):
        if self._closed:
            return
        if self.ptr:
            lib().mlhip_mem_free(self.ptr)
        self._closed = True


class FunctionAttribute(enum.IntEnum):
    """driver.cr:154-165."""
    MaxThreadsPerBlock = 0
    SharedSizeBytes = 1
    ConstSizeBytes = 2
    LocalSizeBytes = 3
    NumRegs = 4
    PtxVersion = 5
    BinaryVersion = 6
    CacheModeCa = 7
    MaxDynamicSharedSizeBytes = 8
    PreferredSharedMemoryCarveout = 9


class KernelFunction:
    """driver.cr:139-152."""

    def __init__(self, handle, name):
        self.handle, self.name = handle, name

    def attribute(self, attr):
        v = ctypes.c_int32()
        check(lib().mlhip_func_get_attribute(ctypes.byref(v), int(attr), self.handle),
              "hipFuncGetAttribute(%s, %s)" % (self.name, FunctionAttribute(attr).name))
        return v.value


class HIPModule:
    """CUDAModule (driver.cr:114-137); the image is a gfx950 code object instead of PTX text."""

    def __init__(self, handle, image):
        self._handle, self._image, self._closed = handle, image, False

    @classmethod
    def load(cls, image, label):
        buf = ctypes.create_string_buffer(bytes(image), len(image))
        h = ctypes.c_void_p()
        check(lib().mlhip_module_load_data(ctypes.byref(h), buf), "hipModuleLoadData(%s)" % label)
        return cls(h, buf)

    @classmethod
    def load_builtin(cls):
        """The code object embedded in libcogni_hip.so (cogni_quant_code_object)."""
        img, size = ctypes.c_void_p(), ctypes.c_size_t()
        check(lib().cogni_quant_code_object(ctypes.byref(img), ctypes.byref(size)), "cogni_quant_code_object")
        return cls.load(ctypes.string_at(img, size.value), "cogni_quant_gfx950")

    def function(self, name):
        fn = ctypes.c_void_p()
        check(lib().mlhip_module_get_function(ctypes.byref(fn), self._handle, name.encode()),
              "hipModuleGetFunction(%s)" % name)
        return KernelFunction(fn, name)

    def close(self):
        if self._closed:
            return
        lib().mlhip_module_unload(self._handle)
        self._closed = True


class HIPGraphExec:
    """driver.cr:228-250."""

    def __init__(self, handle):
        self._handle, self._closed = handle, False

    def launch(self, stream):
        check(lib().mlhip_graph_launch(self._handle, stream.handle), "hipGraphLaunch")

    def upload(self, stream):
        check(lib().mlhip_graph_upload(self._handle, stream.handle), "hipGraphUpload")

    def close(self):
        if self._closed:
            return
        lib().mlhip_graph_exec_destroy(self._handle)
        self._closed = True


class HIPGraph:
    """driver.cr:195-226 (without CUDA's device-launch instantiation, which HIP lacks)."""

    def __init__(self, handle):
        self._handle, self._closed = handle, False

    def instantiate(self):
        ex = ctypes.c_void_p()
        check(lib().mlhip_graph_instantiate(ctypes.byref(ex), self._handle, 0), "hipGraphInstantiateWithFlags")
        return HIPGraphExec(ex)

    def close(self):
        if self._closed:
            return
        lib().mlhip_graph_destroy(self._handle)
        self._closed = True


class HIPStream:
    """driver.cr:167-193. Default priority only."""

    def __init__(self, flags=0):
        self.handle = ctypes.c_void_p()
        check(lib().mlhip_stream_create(ctypes.byref(self.handle), flags), "hipStreamCreate")
        self._closed = False

    def synchronize(self):
        check(lib().mlhip_stream_synchronize(self.handle), "hipStreamSynchronize")

    def begin_capture(self, mode=1):
        check(lib().mlhip_stream_begin_capture(self.handle, mode), "hipStreamBeginCapture")

    def end_capture(self):
        g = ctypes.c_void_p()
        check(lib().mlhip_stream_end_capture(self.handle, ctypes.byref(g)), "hipStreamEndCapture")
        return HIPGraph(g)

    def close(self):
        if self._closed:
            return
        lib().cogni_gemv_release_stream(self.handle)   # the activation image the library may keep for this stream
        lib().mlhip_stream_destroy(self.handle)
        self._closed = True


class Event:
    """GPU-side timestamp on a stream (no counterpart in the reference)."""

    def __init__(self):
        self.handle = ctypes.c_void_p()
        check(lib().mlhip_event_create(ctypes.byref(self.handle)), "hipEventCreate")

    def record(self, stream=None):
        h = stream.handle if stream is not None else current_stream_handle()
        check(lib().mlhip_event_record(self.handle, h), "hipEventRecord")

    def synchronize(self):
        check(lib().mlhip_event_synchronize(self.handle), "hipEventSynchronize")

    def elapsed_ms(self, stop):
        ms = ctypes.c_float()
        check(lib().mlhip_event_elapsed_ms(ctypes.byref(ms), self.handle, stop.handle), "hipEventElapsedTime")
        return ms.value

    def close(self):
        if self.handle:
            lib().mlhip_event_destroy(self.handle)
            self.handle = None


def current_stream_handle():
    return _current_stream


@contextlib.contextmanager
def with_stream(stream):
    """driver.cr:252-260."""
    global _current_stream
    previous = _current_stream
    _current_stream = stream.handle
    try:
        yield
    finally:
        _current_stream = previous


def _host_ptr(buf):
    import numpy as np
    if isinstance(buf, np.ndarray):
        assert buf.flags["C_CONTIGUOUS"]
        return buf.ctypes.data
    return buf


def copy_htod(dst, src, bytesize, what):
    check(lib().mlhip_memcpy_htod(dst, _host_ptr(src), bytesize), "hipMemcpyHtoD(%s)" % what)


def copy_dtoh(dst, src, bytesize, what):
    check(lib().mlhip_memcpy_dtoh(_host_ptr(dst), src, bytesize), "hipMemcpyDtoH(%s)" % what)


def copy_dtod(dst, src, bytesize, what):
    check(lib().mlhip_memcpy_dtod(dst, src, bytesize), "hipMemcpyDtoD(%s)" % what)


def synchronize(what="hipDeviceSynchronize"):
    check(lib().mlhip_ctx_synchronize(), what)


class KernelParams:
    """Boxed kernel arguments kept alive and mutable between launches, the role of the reference's
    heap boxes + @param_keepalive (src/ml/cuda/qwen_full_attn_projection_runner.cr:221-268)."""

    def __init__(self, *boxes):
        self.boxes = list(boxes)
        self.array = (ctypes.c_void_p * len(boxes))(*[ctypes.cast(ctypes.pointer(b), ctypes.c_void_p) for b in boxes])

    def __getitem__(self, i):
        return self.boxes[i]


def launch(fn, grid_x, grid_y, grid_z, block_x, block_y, block_z, params, label, shared_mem_bytes=0):
    """ML::CUDA.launch! (driver.cr:278-286): launches into the current stream."""
    arr = params.array if isinstance(params, KernelParams) else params
    check(lib().mlhip_launch_kernel(fn.handle, grid_x, grid_y, grid_z, block_x, block_y, block_z, shared_mem_bytes,
                                    _current_stream, arr, None), "hipModuleLaunchKernel(%s)" % label)


class ResidentSequenceRunner:
    """driver.cr:288-342: lifecycle facade over caller-supplied closures."""

    def __init__(self, tokens, upload_weights, reset_sequence, run_token, read_outputs=None,
                 run_sequence_override=None):
        if not tokens > 0:
            raise ValueError("tokens must be positive")
        self.tokens = tokens
        self._upload_weights, self._reset_sequence, self._run_token = upload_weights, reset_sequence, run_token
        self._read_outputs, self._run_sequence_override = read_outputs, run_sequence_override
        self._active_tokens = tokens

    @property
    def active_tokens(self):
        return self._active_tokens

    @active_tokens.setter
    def active_tokens(self, value):
        if not value > 0:
            raise ValueError("active_tokens must be positive")
        if not value <= self.tokens:
            raise ValueError("active_tokens must be <= tokens")
        self._active_tokens = value

    def reset_active_tokens(self):
        self._active_tokens = self.tokens

    def upload_weights(self):
        self._upload_weights()

    def reset_sequence(self):
        self._reset_sequence()

    def run_sequence(self):
        if self._run_sequence_override is not None:
            self._run_sequence_override(self._active_tokens)
        else:
            for tok in range(self._active_tokens):
                self._run_token(tok)

    def run_repeated(self, reps):
        if not reps > 0:
            raise ValueError("reps must be positive")
        for _ in range(reps):
            self.run_sequence()
        return reps * self._active_tokens

    def read_outputs(self):
        if self._read_outputs is not None:
            self._read_outputs()
