"""ctypes binding of librmlx_hip.so (the C ABI declared in include/rmlx_hip.h).

This module is plumbing only: it loads the HIP library, declares the prototypes and offers a
thin device-buffer helper.  There is no CPU fallback -- if the library is missing or a call
fails, an exception is raised.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "librmlx_hip.so")

OK, INVALID_SHAPE, NOT_FOUND, RUNTIME_ERROR = 0, 1, 2, 3
F32, F16, BF16, U32, U8 = 0, 1, 2, 3, 4
KERNEL_AUTO, KERNEL_QMV, KERNEL_QMM, KERNEL_GENERIC, KERNEL_QMM_BF16, KERNEL_QMM_LDS, KERNEL_QMV_ROWS = 0, 1, 2, 3, 4, 5, 6
KERNEL_QMM_K2, KERNEL_QMM_RW, KERNEL_QMM_K2_TALL, KERNEL_QMM_K2_FLAT, KERNEL_QMM_K4 = 7, 8, 9, 10, 11
GATHER_AUTO, GATHER_STREAM, GATHER_GEMM, GATHER_PORTABLE = 0, 1, 2, 3  # rmlx_hip_gather_qmm_select kernels
FLOOR_EMPTY, FLOOR_READ4, FLOOR_READ8, FLOOR_MFMA, FLOOR_READ2, FLOOR_MFMA_VALU, FLOOR_LDS, FLOOR_L2_READ = 0, 1, 2, 3, 4, 5, 6, 7  # rmlx_hip_measure_floor kinds


class KernelError(RuntimeError):
    """Mirror of `KernelError` (crates/rmlx-core/src/kernels/mod.rs:29-42)."""

    def __init__(self, code, message):
        super().__init__(message)
        self.code = code
        self.kind = {INVALID_SHAPE: "InvalidShape", NOT_FOUND: "NotFound"}.get(code, "Runtime")


class RmlxArray(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("dtype", ctypes.c_int32), ("ndim", ctypes.c_int32),
                ("shape", ctypes.c_size_t * 4)]


EXPORTS = [
    "rmlx_hip_last_error", "rmlx_hip_init", "rmlx_hip_device_info", "rmlx_hip_malloc", "rmlx_hip_free",
    "rmlx_hip_memset", "rmlx_hip_memcpy_h2d", "rmlx_hip_memcpy_d2h", "rmlx_hip_memcpy_d2d",
    "rmlx_hip_stream_create", "rmlx_hip_stream_sync", "rmlx_hip_stream_destroy", "rmlx_hip_trim_pool", "rmlx_hip_scratch_allocations", "rmlx_hip_graph_begin",
    "rmlx_hip_graph_end", "rmlx_hip_graph_launch", "rmlx_hip_graph_destroy", "rmlx_hip_event_create",
    "rmlx_hip_event_record", "rmlx_hip_event_sync", "rmlx_hip_event_elapsed_ms", "rmlx_hip_event_destroy",
    "rmlx_hip_qweight_create", "rmlx_hip_qweight_destroy", "rmlx_hip_affine_quantized_matmul",
    "rmlx_hip_affine_quantized_matmul_batched", "rmlx_hip_qmm_select", "rmlx_hip_qmm_add_residual", "rmlx_hip_qmm_swiglu", "rmlx_hip_qmm_encode_many", "rmlx_hip_quantized_linear_forward",
    "rmlx_hip_gather_qmm", "rmlx_hip_topk_route", "rmlx_hip_moe_sort", "rmlx_hip_index_gather",
    "rmlx_hip_scatter_weighted_add", "rmlx_hip_silu_gate", "rmlx_hip_expert_group_grouped_forward",
    "rmlx_hip_moe_forward_grouped", "rmlx_hip_moe_forward", "rmlx_hip_moe_forward_noalloc", "rmlx_hip_awq_dequant", "rmlx_hip_gptq_dequant",
    "rmlx_hip_qmm_norm", "rmlx_hip_qweight_set_expert_gemm_min_rows", "rmlx_hip_qweight_set_expert_stream_kernel", "rmlx_hip_qweight_gemm_layout_bytes", "rmlx_hip_qweight_set_gemm_layout", "rmlx_hip_gather_qmm_select", "rmlx_hip_measure_floor",
]

_lib = None


def lib():
    """Load the shared library (raises if it has not been built)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is missing: build it with `make -C rmlx_amd/csrc` "
                           "(or `python -c 'import __graft_entry__ as g; g.build()'`)")
    L = ctypes.CDLL(LIB_PATH)
    vp, sz, i32, u32 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int32, ctypes.c_uint32
    arr = ctypes.POINTER(RmlxArray)
    L.rmlx_hip_last_error.restype = ctypes.c_char_p
    L.rmlx_hip_last_error.argtypes = []
    protos = {
        "rmlx_hip_init": [i32],
        "rmlx_hip_device_info": [ctypes.POINTER(ctypes.c_int64)],
        "rmlx_hip_malloc": [ctypes.POINTER(vp), sz],
        "rmlx_hip_free": [vp],
        "rmlx_hip_memset": [vp, i32, sz, vp],
        "rmlx_hip_memcpy_h2d": [vp, vp, sz, vp],
        "rmlx_hip_memcpy_d2h": [vp, vp, sz, vp],
        "rmlx_hip_memcpy_d2d": [vp, vp, sz, vp],
        "rmlx_hip_stream_create": [ctypes.POINTER(vp)],
        "rmlx_hip_stream_sync": [vp],
        "rmlx_hip_stream_destroy": [vp],
        "rmlx_hip_trim_pool": [vp],
        "rmlx_hip_measure_floor": [i32, vp, sz, sz, u32, vp, sz, vp],
        "rmlx_hip_graph_begin": [vp],
        "rmlx_hip_graph_end": [vp, ctypes.POINTER(vp)],
        "rmlx_hip_graph_launch": [vp, vp],
        "rmlx_hip_graph_destroy": [vp],
        "rmlx_hip_event_create": [ctypes.POINTER(vp)],
        "rmlx_hip_event_record": [vp, vp],
        "rmlx_hip_event_sync": [vp],
        "rmlx_hip_event_elapsed_ms": [vp, vp, ctypes.POINTER(ctypes.c_float)],
        "rmlx_hip_event_destroy": [vp],
        "rmlx_hip_qweight_create": [vp, sz, vp, sz, vp, sz, u32, u32, sz, sz, sz, ctypes.POINTER(vp)],
        "rmlx_hip_qweight_destroy": [vp],
        "rmlx_hip_affine_quantized_matmul": [vp, arr, vp, sz, vp],
        "rmlx_hip_affine_quantized_matmul_batched": [vp, arr, vp, sz, vp],
        "rmlx_hip_qmm_select": [vp, arr, i32, vp, sz, vp],
        "rmlx_hip_qmm_add_residual": [vp, arr, arr, vp, sz, vp],
        "rmlx_hip_qmm_swiglu": [vp, arr, arr, vp, sz, vp],
        "rmlx_hip_qmm_encode_many": [ctypes.POINTER(vp), sz, arr, ctypes.POINTER(vp), sz, sz, sz, i32, vp],
        "rmlx_hip_quantized_linear_forward": [vp, arr, vp, vp, sz, vp],
        "rmlx_hip_gather_qmm": [arr, vp, sz, vp, sz, vp, sz, arr, sz, sz, sz, sz, sz, u32, vp, sz, vp],
        "rmlx_hip_gather_qmm_select": [arr, vp, sz, vp, sz, vp, sz, arr, sz, sz, sz, sz, sz, u32, i32, vp, sz, vp],
        "rmlx_hip_topk_route": [arr, sz, arr, i32, vp, vp, vp, vp, vp],
        "rmlx_hip_moe_sort": [vp, sz, sz, vp, vp, vp],
        "rmlx_hip_index_gather": [vp, sz, sz, vp, sz, vp, vp],
        "rmlx_hip_scatter_weighted_add": [vp, sz, sz, vp, vp, vp, sz, vp],
        "rmlx_hip_silu_gate": [vp, vp, vp, sz, vp],
        "rmlx_hip_expert_group_grouped_forward": [vp, vp, vp, sz, vp, vp, arr, vp, sz, vp],
        "rmlx_hip_moe_forward_grouped": [vp, vp, vp, arr, vp, vp, sz, vp, sz, vp],
        "rmlx_hip_moe_forward": [vp, vp, vp, arr, arr, sz, arr, vp, sz, vp],
        "rmlx_hip_moe_forward_noalloc": [vp, vp, vp, arr, arr, sz, arr, vp, sz, vp],
        "rmlx_hip_qmm_norm": [vp, arr, arr, arr, vp, sz, vp],
        "rmlx_hip_awq_dequant": [vp, sz, vp, sz, vp, sz, sz, sz, sz, vp, sz, vp],
        "rmlx_hip_gptq_dequant": [vp, sz, vp, sz, vp, sz, vp, sz, sz, sz, sz, vp, sz, vp],
    }
    for name, argtypes in protos.items():
        fn = getattr(L, name)
        fn.argtypes = argtypes
        fn.restype = i32
    L.rmlx_hip_qweight_set_expert_gemm_min_rows.argtypes = [vp, u32]
    L.rmlx_hip_qweight_set_expert_gemm_min_rows.restype = u32
    L.rmlx_hip_qweight_set_expert_stream_kernel.argtypes = [vp, u32]
    L.rmlx_hip_qweight_set_expert_stream_kernel.restype = u32
    L.rmlx_hip_qweight_gemm_layout_bytes.argtypes = [vp]
    L.rmlx_hip_qweight_gemm_layout_bytes.restype = ctypes.c_size_t
    L.rmlx_hip_qweight_set_gemm_layout.argtypes = [vp, vp, ctypes.c_size_t, vp]
    L.rmlx_hip_qweight_set_gemm_layout.restype = ctypes.c_int32
    L.rmlx_hip_scratch_allocations.argtypes = []
    L.rmlx_hip_scratch_allocations.restype = ctypes.c_uint64
    _lib = L
    return L


def check(status):
    if status != OK:
        raise KernelError(status, lib().rmlx_hip_last_error().decode())


_initialised = False


def init(device=0):
    global _initialised
    check(lib().rmlx_hip_init(device))
    _initialised = True


def scratch_allocations():
    """Device allocations the library's scratch pool has made so far in this process."""
    return int(lib().rmlx_hip_scratch_allocations())


def device_info():
    out = (ctypes.c_int64 * 8)()
    check(lib().rmlx_hip_device_info(out))
    keys = ["compute_units", "wavefront", "lds_per_block", "global_mem_mib", "clock_khz", "mem_clock_khz",
            "bus_width_bits", "l2_bytes"]
    return dict(zip(keys, list(out)))


_NP_DTYPE = {F32: np.float32, F16: np.float16, BF16: np.uint16, U32: np.uint32, U8: np.uint8}


class DeviceBuffer:
    """A hipMalloc'ed buffer with a shape and an rmlx dtype tag (bf16 travels as uint16 bits)."""

    def __init__(self, shape, dtype):
        self.shape = tuple(int(s) for s in shape)
        self.dtype = dtype
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * np.dtype(_NP_DTYPE[dtype]).itemsize
        p = ctypes.c_void_p()
        check(lib().rmlx_hip_malloc(ctypes.byref(p), self.nbytes))
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a, dtype=None):
        a = np.ascontiguousarray(a)
        if dtype is None:
            dtype = {np.dtype(np.float32): F32, np.dtype(np.float16): F16, np.dtype(np.uint32): U32,
                     np.dtype(np.uint8): U8}[a.dtype]
        assert a.dtype == np.dtype(_NP_DTYPE[dtype]), (a.dtype, dtype)
        buf = cls(a.shape, dtype)
        check(lib().rmlx_hip_memcpy_h2d(buf.ptr, a.ctypes.data, buf.nbytes, None))
        return buf

    def numpy(self):
        out = np.empty(self.shape, _NP_DTYPE[self.dtype])
        check(lib().rmlx_hip_memcpy_d2h(out.ctypes.data, self.ptr, self.nbytes, None))
        return out

    def array(self, shape=None, offset_elems=0):
        """The rmlx_array view handed to the C ABI."""
        shape = self.shape if shape is None else tuple(shape)
        a = RmlxArray()
        a.data = self.ptr + offset_elems * np.dtype(_NP_DTYPE[self.dtype]).itemsize
        a.dtype = self.dtype
        a.ndim = len(shape)
        for i, s in enumerate(shape):
            a.shape[i] = s
        return a

    def free(self):
        if self.ptr:
            lib().rmlx_hip_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Stream:
    def __init__(self):
        p = ctypes.c_void_p()
        check(lib().rmlx_hip_stream_create(ctypes.byref(p)))
        self.handle = p.value

    def sync(self):
        check(lib().rmlx_hip_stream_sync(self.handle))

    def __del__(self):
        try:
            if self.handle:
                lib().rmlx_hip_stream_destroy(self.handle)
        except Exception:
            pass


class Graph:
    """A recorded train of calls on a stream: `with Graph.record(stream) as g: ...calls...`, then `g.launch(stream)`."""

    def __init__(self, stream):
        self.stream, self.handle = stream, None

    @classmethod
    def record(cls, stream):
        return cls(stream)

    def __enter__(self):
        check(lib().rmlx_hip_graph_begin(self.stream.handle))
        return self

    def __exit__(self, exc_type, exc, tb):
        p = ctypes.c_void_p()
        status = lib().rmlx_hip_graph_end(self.stream.handle, ctypes.byref(p))
        if exc_type is None:
            check(status)
            self.handle = p.value
        return False

    def launch(self, stream=None):
        check(lib().rmlx_hip_graph_launch(self.handle, (stream or self.stream).handle))

    def __del__(self):
        try:
            if self.handle:
                lib().rmlx_hip_graph_destroy(self.handle)
        except Exception:
            pass


class Event:
    def __init__(self):
        p = ctypes.c_void_p()
        check(lib().rmlx_hip_event_create(ctypes.byref(p)))
        self.handle = p.value

    def record(self, stream=None):
        check(lib().rmlx_hip_event_record(self.handle, stream.handle if stream else None))

    def sync(self):
        check(lib().rmlx_hip_event_sync(self.handle))

    def elapsed_ms(self, later):
        ms = ctypes.c_float()
        check(lib().rmlx_hip_event_elapsed_ms(self.handle, later.handle, ctypes.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            if self.handle:
                lib().rmlx_hip_event_destroy(self.handle)
        except Exception:
            pass
