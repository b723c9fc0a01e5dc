"""ctypes binding of the C-ABI in ``include/thip.h``.

Host-side glue only: everything that computes lives in ``libthip.so``.  There is
no CPU fallback; if the library or a gfx950 device is missing the calls raise.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libthip.so")

# status codes (include/thip.h)
OK = 0
INVALID_ARGUMENT = 3
RESOURCE_EXHAUSTED = 8
FAILED_PRECONDITION = 9
OUT_OF_RANGE = 11
UNIMPLEMENTED = 12
INTERNAL = 13
UNAVAILABLE = 14

STATUS_NAMES = {
    OK: "OK", INVALID_ARGUMENT: "INVALID_ARGUMENT", RESOURCE_EXHAUSTED: "RESOURCE_EXHAUSTED",
    FAILED_PRECONDITION: "FAILED_PRECONDITION", OUT_OF_RANGE: "OUT_OF_RANGE",
    UNIMPLEMENTED: "UNIMPLEMENTED", INTERNAL: "INTERNAL", UNAVAILABLE: "UNAVAILABLE",
}

DTYPE_I8, DTYPE_I16, DTYPE_I32, DTYPE_BF16, DTYPE_F32, DTYPE_I1 = 1, 2, 3, 4, 5, 6
# numpy has no bfloat16: uint16 arrays carry bf16 bit patterns; uint8 arrays of 0 / 1 carry i1 truth values
_NP_TO_DTYPE = {np.dtype(np.int8): DTYPE_I8, np.dtype(np.int16): DTYPE_I16, np.dtype(np.int32): DTYPE_I32,
                np.dtype(np.uint16): DTYPE_BF16, np.dtype(np.float32): DTYPE_F32, np.dtype(np.uint8): DTYPE_I1}
_DTYPE_TO_NP = {v: k for k, v in _NP_TO_DTYPE.items()}

BINDING_HOST, BINDING_DEVICE = 0, 1

# every symbol include/thip.h declares
EXPORTED_SYMBOLS = [
    "thip_status_message", "thip_version", "thip_descriptor_version",
    "thip_program_create", "thip_program_destroy", "thip_program_set_name", "thip_program_binding", "thip_program_constant",
    "thip_program_tensor", "thip_program_view", "thip_gemm_tile_choice", "thip_hl_conv2d", "thip_hl_depthwise_conv2d", "thip_hl_fully_connected",
    "thip_hl_matmul", "thip_hl_maxpool2d", "thip_hl_avg_pool2d", "thip_hl_add", "thip_hl_transpose", "thip_hl_expand_weights",
    "thip_hl_fma", "thip_hl_mul", "thip_hl_act", "thip_hl_elementwisebinary", "thip_hl_elementwiseunary", "thip_hl_elementwiseshift", "thip_hl_table",
    "thip_program_serialize", "thip_blob_free",
    "thip_device_create", "thip_device_destroy", "thip_device_name", "thip_device_alloc",
    "thip_device_free", "thip_device_h2d", "thip_device_d2h", "thip_device_synchronize",
    "thip_device_set_event_log", "thip_device_set_dump_dirs", "thip_device_mfma_rate", "thip_device_stream_floor", "thip_device_stream_floor_tuned", "thip_infer_format", "thip_descriptor_validate", "thip_descriptor_info", "thip_descriptor_binding", "thip_descriptor_segment",
    "thip_executable_create", "thip_executable_destroy", "thip_executable_run",
    "thip_executable_enqueue", "thip_executable_enqueue_noalloc", "thip_executable_wait", "thip_executable_set_wait_timeout", "thip_executable_time", "thip_executable_time_rotating",
    "thip_executable_op_count", "thip_executable_op_kernel", "thip_executable_binding_count",
    "thip_executable_binding_size",
]


class ThipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("%s: %s" % (STATUS_NAMES.get(code, str(code)), message))
        self.code = code
        self.message = message


class DescriptorInfo(ctypes.Structure):
    _fields_ = [("executable_name", ctypes.c_char * 64), ("runtime_version", ctypes.c_uint32), ("hw_id", ctypes.c_uint32),
                ("action_count", ctypes.c_uint32), ("binding_count", ctypes.c_uint32), ("segment_count", ctypes.c_uint32),
                ("intermediate_count", ctypes.c_uint32), ("intermediate_bytes", ctypes.c_uint64), ("total_size", ctypes.c_uint64)]


class BindingInfo(ctypes.Structure):
    _fields_ = [("id", ctypes.c_uint32), ("address", ctypes.c_uint64), ("offset", ctypes.c_uint64), ("size", ctypes.c_uint64),
                ("is_read_only", ctypes.c_uint8), ("is_write_only", ctypes.c_uint8), ("is_used", ctypes.c_uint8)]


class SegmentInfo(ctypes.Structure):
    _fields_ = [("address", ctypes.c_uint64), ("size", ctypes.c_uint64), ("data", ctypes.POINTER(ctypes.c_uint8))]


def describe_blob(blob):
    """What a descriptor blob holds in the terms of the reference's executable schema: (info, bindings, segments)."""
    buf = ctypes.create_string_buffer(bytes(blob), len(blob))
    info = DescriptorInfo()
    check(lib().thip_descriptor_info(buf, len(blob), ctypes.byref(info)))
    bindings, segments = [], []
    for i in range(info.binding_count):
        b = BindingInfo()
        check(lib().thip_descriptor_binding(buf, len(blob), i, ctypes.byref(b)))
        bindings.append(dict(id=b.id, address=b.address, offset=b.offset, size=b.size, is_read_only=bool(b.is_read_only),
                             is_write_only=bool(b.is_write_only), is_used=bool(b.is_used)))
    for i in range(info.segment_count):
        s = SegmentInfo()
        check(lib().thip_descriptor_segment(buf, len(blob), i, ctypes.byref(s)))
        segments.append(dict(address=s.address, size=s.size, data=bytes(ctypes.string_at(s.data, s.size))))
    return dict(executable_name=info.executable_name.decode(), runtime_version=info.runtime_version, hw_id=info.hw_id,
                action_count=info.action_count, intermediate_count=info.intermediate_count, intermediate_bytes=info.intermediate_bytes,
                total_size=info.total_size), bindings, segments


class DispatchState(ctypes.Structure):
    _fields_ = [
        ("constant_count", ctypes.c_uint32),
        ("constants", ctypes.POINTER(ctypes.c_uint32)),
        ("binding_count", ctypes.c_uint32),
        ("binding_ptrs", ctypes.POINTER(ctypes.c_void_p)),
        ("binding_lengths", ctypes.POINTER(ctypes.c_size_t)),
        ("binding_flags", ctypes.POINTER(ctypes.c_uint8)),
    ]


class HlConv2d(ctypes.Structure):
    _fields_ = [
        ("init", ctypes.c_int32), ("input_zp", ctypes.c_int32), ("weight_zp", ctypes.c_int32),
        ("output_zp", ctypes.c_int32), ("output_min", ctypes.c_int32), ("output_max", ctypes.c_int32),
        ("shift_factor", ctypes.c_int32), ("groups", ctypes.c_int32),
        ("pad", ctypes.c_int64 * 4), ("stride", ctypes.c_int64 * 2), ("dilation", ctypes.c_int64 * 2),
        ("vectorization_mode", ctypes.c_int32), ("weights", ctypes.c_int32),
        ("scale_bias", ctypes.c_int32), ("input", ctypes.c_int32),
        ("nhwc_input", ctypes.c_int32), ("segment_output", ctypes.c_int32),
    ]


class HlDepthwiseConv2d(ctypes.Structure):
    _fields_ = HlConv2d._fields_ + [("is_dw1d_stride1", ctypes.c_int32)]


class HlFullyConnected(ctypes.Structure):
    _fields_ = [
        ("init", ctypes.c_int32), ("input_zp", ctypes.c_int32), ("weight_zp", ctypes.c_int32),
        ("output_zp", ctypes.c_int32), ("output_min", ctypes.c_int32), ("output_max", ctypes.c_int32),
        ("shift_factor", ctypes.c_int32), ("vectorization_mode", ctypes.c_int32),
        ("weights", ctypes.c_int32), ("scale_bias", ctypes.c_int32), ("input", ctypes.c_int32),
    ]


class HlMatmul(ctypes.Structure):
    _fields_ = [
        ("init", ctypes.c_int32), ("output_zp", ctypes.c_int32), ("output_min", ctypes.c_int32),
        ("output_max", ctypes.c_int32), ("shift", ctypes.c_int32), ("scale_bias", ctypes.c_int32),
        ("input1", ctypes.c_int32), ("input2", ctypes.c_int32),
    ]


class HlMaxPool2d(ctypes.Structure):
    _fields_ = [
        ("init", ctypes.c_int32), ("input_zp", ctypes.c_int32), ("output_min", ctypes.c_int32),
        ("output_max", ctypes.c_int32), ("stride", ctypes.c_int64 * 2), ("pad", ctypes.c_int64 * 4),
        ("kernel", ctypes.c_int64 * 2), ("weights", ctypes.c_int32), ("scale_bias", ctypes.c_int32),
        ("input", ctypes.c_int32), ("segment_output", ctypes.c_int32), ("nhwc_input", ctypes.c_int32),
    ]


class HlAvgPool2d(ctypes.Structure):
    _fields_ = [
        ("init", ctypes.c_int32), ("input_zp", ctypes.c_int32), ("output_zp", ctypes.c_int32),
        ("output_min", ctypes.c_int32), ("output_max", ctypes.c_int32), ("shift_factor", ctypes.c_int32),
        ("weights", ctypes.c_int32), ("scale_bias", ctypes.c_int32), ("input", ctypes.c_int32),
    ]


class HlExpandWeights(ctypes.Structure):
    _fields_ = [
        ("init", ctypes.c_int32), ("scale_bias", ctypes.c_int32), ("output_min", ctypes.c_int32),
        ("output_max", ctypes.c_int32), ("scale", ctypes.c_int32), ("input", ctypes.c_int32),
        ("block_size", ctypes.c_int32),
    ]


class HlFma(ctypes.Structure):
    _fields_ = [
        ("init", ctypes.c_int32), ("output_zp", ctypes.c_int32), ("output_min", ctypes.c_int32),
        ("output_max", ctypes.c_int32), ("shift_factor", ctypes.c_int32), ("weights", ctypes.c_int32),
        ("scale_bias", ctypes.c_int32), ("input", ctypes.c_int32),
    ]


class HlMul(ctypes.Structure):
    _fields_ = [
        ("init", ctypes.c_int32), ("output_zp", ctypes.c_int32), ("output_min", ctypes.c_int32),
        ("output_max", ctypes.c_int32), ("scale_bias", ctypes.c_int32), ("shift", ctypes.c_int32),
        ("input1", ctypes.c_int32), ("input2", ctypes.c_int32),
    ]


class HlElementwiseUnary(ctypes.Structure):
    _fields_ = [("init", ctypes.c_int32), ("op_type", ctypes.c_int32), ("input", ctypes.c_int32)]


class HlTable(ctypes.Structure):
    _fields_ = [("init", ctypes.c_int32), ("scale_bias", ctypes.c_int32), ("input", ctypes.c_int32), ("dynamic_table", ctypes.c_int32),
                ("static_table", ctypes.POINTER(ctypes.c_int32)), ("static_table_count", ctypes.c_int32)]


class HlElementwiseShift(ctypes.Structure):
    _fields_ = [("init", ctypes.c_int32), ("op_type", ctypes.c_int32), ("round", ctypes.c_int32), ("input1", ctypes.c_int32),
                ("input2", ctypes.c_int32)]


class HlAct(ctypes.Structure):
    _fields_ = [
        ("init", ctypes.c_int32), ("name", ctypes.c_char_p), ("input_zp", ctypes.c_int32),
        ("output_zp", ctypes.c_int32), ("min_int", ctypes.c_int64), ("max_int", ctypes.c_int64),
        ("min_fp", ctypes.c_float), ("max_fp", ctypes.c_float), ("input", ctypes.c_int32),
        ("weights", ctypes.c_int32),
    ]


class HlElementwiseBinary(ctypes.Structure):
    _fields_ = [
        ("init", ctypes.c_int32), ("op_type", ctypes.c_int32), ("input1", ctypes.c_int32), ("input2", ctypes.c_int32),
        ("is_unsigned", ctypes.c_int32),
    ]


NO_VALUE = -1
# torq_hl.elementwisebinary op_type values on this path (the reference's ElementwiseOpEnum)
BITWISE_AND, BITWISE_OR, BITWISE_XOR, MINIMUM, MAXIMUM = 0, 1, 2, 4, 5


class HlAdd(ctypes.Structure):
    _fields_ = [
        ("init", ctypes.c_int32), ("name", ctypes.c_char_p), ("input_zp", ctypes.c_int32),
        ("output_zp", ctypes.c_int32), ("output_min", ctypes.c_int32), ("output_max", ctypes.c_int32),
        ("shift_factor", ctypes.c_int32), ("weights", ctypes.c_int32), ("scale_bias", ctypes.c_int32),
        ("input1", ctypes.c_int32), ("input2", ctypes.c_int32), ("segment_output", ctypes.c_int32),
        ("rhs_is_scalar", ctypes.c_int32),
    ]


class HlTranspose(ctypes.Structure):
    _fields_ = [
        ("init", ctypes.c_int32), ("rank", ctypes.c_int32), ("perm", ctypes.c_int64 * 4),
        ("input", ctypes.c_int32),
    ]


_lib = None


def library_built():
    return os.path.exists(LIB_PATH)


def lib():
    """Loads ``libthip.so``; raises if it has not been built (no fallback)."""
    global _lib
    if _lib is not None:
        return _lib
    if not library_built():
        raise ThipError(UNAVAILABLE, "%s is missing: run `python torq-compiler_amd/build.py` "
                                     "(or __graft_entry__.build()) first" % LIB_PATH)
    L = ctypes.CDLL(LIB_PATH)
    L.thip_status_message.restype = ctypes.c_char_p
    L.thip_version.restype = ctypes.c_uint32
    L.thip_descriptor_version.restype = ctypes.c_uint32
    vp, i32, u32, sz = ctypes.c_void_p, ctypes.c_int32, ctypes.c_uint32, ctypes.c_size_t
    P = ctypes.POINTER
    L.thip_program_create.argtypes = [P(vp)]
    L.thip_program_destroy.argtypes = [vp]
    L.thip_program_destroy.restype = None
    L.thip_program_binding.argtypes = [vp, u32, i32, i32, P(ctypes.c_int64), P(i32)]
    L.thip_program_constant.argtypes = [vp, i32, i32, P(ctypes.c_int64), vp, sz, P(i32)]
    L.thip_program_tensor.argtypes = [vp, i32, i32, P(ctypes.c_int64), P(i32)]
    L.thip_program_view.argtypes = [vp, i32, ctypes.c_int64, i32, P(ctypes.c_int64), P(i32)]
    L.thip_gemm_tile_choice.argtypes = [i32, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, i32, i32, P(ctypes.c_uint32), ctypes.c_char_p, ctypes.c_size_t]
    for name, st in [("thip_hl_conv2d", HlConv2d), ("thip_hl_depthwise_conv2d", HlDepthwiseConv2d),
                     ("thip_hl_fully_connected", HlFullyConnected), ("thip_hl_matmul", HlMatmul),
                     ("thip_hl_maxpool2d", HlMaxPool2d), ("thip_hl_avg_pool2d", HlAvgPool2d),
                     ("thip_hl_add", HlAdd), ("thip_hl_transpose", HlTranspose),
                     ("thip_hl_expand_weights", HlExpandWeights), ("thip_hl_fma", HlFma), ("thip_hl_mul", HlMul),
                     ("thip_hl_act", HlAct), ("thip_hl_elementwisebinary", HlElementwiseBinary)]:
        getattr(L, name).argtypes = [vp, P(st)]
    L.thip_program_serialize.argtypes = [vp, P(vp), P(sz)]
    L.thip_blob_free.argtypes = [vp]
    L.thip_blob_free.restype = None
    L.thip_device_create.argtypes = [i32, P(vp)]
    L.thip_device_destroy.argtypes = [vp]
    L.thip_device_destroy.restype = None
    L.thip_device_name.argtypes = [vp, ctypes.c_char_p, sz]
    L.thip_device_alloc.argtypes = [vp, sz, P(vp)]
    L.thip_device_free.argtypes = [vp, vp]
    L.thip_device_h2d.argtypes = [vp, vp, vp, sz]
    L.thip_device_d2h.argtypes = [vp, vp, vp, sz]
    L.thip_device_synchronize.argtypes = [vp]
    L.thip_device_set_event_log.argtypes = [vp, ctypes.c_char_p]
    L.thip_device_set_dump_dirs.argtypes = [vp, ctypes.c_char_p, ctypes.c_char_p]
    L.thip_device_mfma_rate.argtypes = [vp, i32, i32, i32, P(ctypes.c_double)]
    L.thip_device_stream_floor.argtypes = [vp, i32, sz, i32, P(ctypes.c_double)]
    L.thip_device_stream_floor_tuned.argtypes = [vp, i32, sz, i32, P(ctypes.c_double), ctypes.c_char_p, sz]
    L.thip_infer_format.argtypes = [vp, sz, sz, ctypes.c_char_p, P(sz)]
    L.thip_descriptor_validate.argtypes = [vp, sz]
    L.thip_descriptor_info.argtypes = [vp, sz, vp]
    L.thip_descriptor_binding.argtypes = [vp, sz, u32, vp]
    L.thip_descriptor_segment.argtypes = [vp, sz, u32, vp]
    L.thip_program_set_name.argtypes = [vp, ctypes.c_char_p]
    L.thip_executable_create.argtypes = [vp, vp, sz, P(u32), sz, P(vp)]
    L.thip_executable_destroy.argtypes = [vp]
    L.thip_executable_destroy.restype = None
    L.thip_executable_run.argtypes = [vp, P(DispatchState)]
    L.thip_executable_enqueue.argtypes = [vp, P(DispatchState)]
    L.thip_executable_enqueue_noalloc.argtypes = [vp, P(DispatchState)]
    L.thip_executable_wait.argtypes = [vp]
    L.thip_executable_set_wait_timeout.argtypes = [vp, ctypes.c_int64]
    L.thip_executable_time.argtypes = [vp, P(DispatchState), i32, P(ctypes.c_float)]
    L.thip_executable_time_rotating.argtypes = [vp, P(DispatchState), u32, i32, P(ctypes.c_float)]
    L.thip_executable_op_count.argtypes = [vp, P(u32)]
    L.thip_executable_op_kernel.argtypes = [vp, u32, ctypes.c_char_p, sz]
    L.thip_executable_binding_count.argtypes = [vp, P(u32)]
    L.thip_executable_binding_size.argtypes = [vp, u32, P(sz)]
    _lib = L
    return L


def check(code):
    if code != OK:
        raise ThipError(code, lib().thip_status_message().decode("utf-8", "replace"))


def _shape_array(shape):
    return (ctypes.c_int64 * len(shape))(*[int(s) for s in shape])


class Device:
    """A gfx950 GPU (thip_device_t)."""

    def __init__(self, ordinal=0):
        self._h = ctypes.c_void_p()
        check(lib().thip_device_create(int(ordinal), ctypes.byref(self._h)))

    @property
    def handle(self):
        return self._h

    def name(self):
        buf = ctypes.create_string_buffer(64)
        check(lib().thip_device_name(self._h, buf, 64))
        return buf.value.decode()

    def alloc(self, size):
        p = ctypes.c_void_p()
        check(lib().thip_device_alloc(self._h, int(size), ctypes.byref(p)))
        return p.value

    def free(self, ptr):
        check(lib().thip_device_free(self._h, ctypes.c_void_p(ptr)))

    def upload(self, array):
        """Copies a numpy array into new device memory; returns the device pointer."""
        a = np.ascontiguousarray(array)
        p = self.alloc(max(a.nbytes, 1))
        check(lib().thip_device_h2d(self._h, ctypes.c_void_p(p), a.ctypes.data_as(ctypes.c_void_p), a.nbytes))
        return p

    def download(self, ptr, shape, dtype):
        out = np.empty(shape, dtype=dtype)
        check(lib().thip_device_d2h(self._h, out.ctypes.data_as(ctypes.c_void_p), ctypes.c_void_p(ptr), out.nbytes))
        return out

    def synchronize(self):
        check(lib().thip_device_synchronize(self._h))

    def set_event_log(self, path):
        check(lib().thip_device_set_event_log(self._h, path.encode() if path else None))

    def mfma_rate(self, random_operands, workgroups=256, iterations=10000):
        """Sustained int8 MFMA rate in TOP/s of `workgroups` workgroups doing nothing else (benchmark calibration)."""
        tops = ctypes.c_double()
        check(lib().thip_device_mfma_rate(self._h, int(bool(random_operands)), int(workgroups), int(iterations), ctypes.byref(tops)))
        return tops.value

    def stream_floor(self, reads_per_write, write_bytes, cold=True, variant=False):
        """Microseconds per launch of the fastest streaming kernel with next to no arithmetic (benchmark calibration);
        variant=True: (microseconds, name of the winning kernel)."""
        us = ctypes.c_double()
        name = ctypes.create_string_buffer(64)
        check(lib().thip_device_stream_floor_tuned(self._h, int(reads_per_write), int(write_bytes), int(bool(cold)), ctypes.byref(us), name, 64))
        return (us.value, name.value.decode()) if variant else us.value

    def set_dump_dirs(self, io_data_dir=None, buffers_dir=None):
        """Debug dumps of the bindings of blocking dispatches / of every buffer a kernel record wrote (None: off)."""
        check(lib().thip_device_set_dump_dirs(self._h, io_data_dir.encode() if io_data_dir else None,
                                              buffers_dir.encode() if buffers_dir else None))

    def close(self):
        if self._h:
            lib().thip_device_destroy(self._h)
            self._h = ctypes.c_void_p()


def infer_format(blob):
    buf = ctypes.create_string_buffer(32)
    size = ctypes.c_size_t(0)
    check(lib().thip_infer_format(blob, len(blob), 32, buf, ctypes.byref(size)))
    return buf.value.decode(), size.value


ADDRESSING_DENSE, ADDRESSING_GATHER, ADDRESSING_RUNS, ADDRESSING_WINDOW = 0, 1, 2, 3


def gemm_tile_choice(addressing, M, N, K, C=1, out_dtype=1, add_follows=False):
    """(tile number, tile name) the serialiser gives an integer GEMM-shaped op of this geometry (thip_gemm_tile_choice)."""
    v = ctypes.c_uint32()
    buf = ctypes.create_string_buffer(64)
    check(lib().thip_gemm_tile_choice(int(addressing), int(M), int(N), int(K), int(C), int(out_dtype), int(bool(add_follows)), ctypes.byref(v), buf, 64))
    return v.value, buf.value.decode()


def make_state(ptrs, lengths, flags, constants=None):
    """Builds a thip_dispatch_state_t; returns (state, keepalive)."""
    n = len(ptrs)
    ptr_arr = (ctypes.c_void_p * max(n, 1))(*[ctypes.c_void_p(p) for p in ptrs])
    len_arr = (ctypes.c_size_t * max(n, 1))(*[int(l) for l in lengths])
    flag_arr = (ctypes.c_uint8 * max(n, 1))(*[int(f) for f in flags])
    st = DispatchState()
    if constants is not None and len(constants):
        c = np.ascontiguousarray(constants, dtype=np.uint32)
        st.constant_count = c.size
        st.constants = c.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32))
    else:
        c = None
        st.constant_count = 0
        st.constants = None
    st.binding_count = n
    st.binding_ptrs = ctypes.cast(ptr_arr, ctypes.POINTER(ctypes.c_void_p))
    st.binding_lengths = ctypes.cast(len_arr, ctypes.POINTER(ctypes.c_size_t))
    st.binding_flags = ctypes.cast(flag_arr, ctypes.POINTER(ctypes.c_uint8))
    return st, (ptr_arr, len_arr, flag_arr, c)


class Executable:
    """A loaded dispatch descriptor (thip_executable_t)."""

    def __init__(self, device, blob, constants=None):
        self.device = device
        self._h = ctypes.c_void_p()
        cptr, ccount = None, 0
        if constants is not None and len(constants):
            self._constants = np.ascontiguousarray(constants, dtype=np.uint32)
            cptr = self._constants.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32))
            ccount = self._constants.size
        check(lib().thip_executable_create(device.handle, blob, len(blob), cptr, ccount, ctypes.byref(self._h)))

    def op_kernels(self):
        n = ctypes.c_uint32()
        check(lib().thip_executable_op_count(self._h, ctypes.byref(n)))
        names = []
        for i in range(n.value):
            buf = ctypes.create_string_buffer(64)
            check(lib().thip_executable_op_kernel(self._h, i, buf, 64))
            names.append(buf.value.decode())
        return names

    def binding_sizes(self):
        n = ctypes.c_uint32()
        check(lib().thip_executable_binding_count(self._h, ctypes.byref(n)))
        sizes = []
        for i in range(n.value):
            s = ctypes.c_size_t()
            check(lib().thip_executable_binding_size(self._h, i, ctypes.byref(s)))
            sizes.append(s.value)
        return sizes

    def run_host(self, arrays):
        """Blocking dispatch on host numpy arrays (inputs and outputs, in binding order)."""
        ptrs = [a.ctypes.data for a in arrays]
        st, keep = make_state(ptrs, [a.nbytes for a in arrays], [BINDING_HOST] * len(arrays))
        check(lib().thip_executable_run(self._h, ctypes.byref(st)))
        del keep

    def run_device(self, ptrs, lengths):
        st, keep = make_state(ptrs, lengths, [BINDING_DEVICE] * len(ptrs))
        check(lib().thip_executable_run(self._h, ctypes.byref(st)))
        del keep

    def run_state(self, state):
        check(lib().thip_executable_run(self._h, ctypes.byref(state)))

    def enqueue_device(self, ptrs, lengths):
        st, keep = make_state(ptrs, lengths, [BINDING_DEVICE] * len(ptrs))
        check(lib().thip_executable_enqueue(self._h, ctypes.byref(st)))
        del keep

    def enqueue_device_noalloc(self, ptrs, lengths):
        """thip_executable_enqueue_noalloc: the dispatch without any device allocation (scratch from the static array)."""
        st, keep = make_state(ptrs, lengths, [BINDING_DEVICE] * len(ptrs))
        check(lib().thip_executable_enqueue_noalloc(self._h, ctypes.byref(st)))
        del keep

    def wait(self):
        check(lib().thip_executable_wait(self._h))

    def set_wait_timeout(self, milliseconds):
        """Waits for the GPU give up after this long (THIP_INTERNAL; the executable is abandoned); <= 0: no limit."""
        check(lib().thip_executable_set_wait_timeout(self._h, int(milliseconds)))

    def time_device(self, ptrs, lengths, iterations):
        """Mean milliseconds per dispatch over `iterations`, HIP events on the executable's stream."""
        st, keep = make_state(ptrs, lengths, [BINDING_DEVICE] * len(ptrs))
        ms = ctypes.c_float()
        check(lib().thip_executable_time(self._h, ctypes.byref(st), int(iterations), ctypes.byref(ms)))
        del keep
        return ms.value

    def time_device_rotating(self, ptr_sets, lengths, iterations):
        """Like time_device, with dispatch i on ptr_sets[i % len(ptr_sets)] (a working set larger than the caches)."""
        made = [make_state(ptrs, lengths, [BINDING_DEVICE] * len(ptrs)) for ptrs in ptr_sets]
        states = (DispatchState * len(made))(*[m[0] for m in made])
        ms = ctypes.c_float()
        check(lib().thip_executable_time_rotating(self._h, states, len(made), int(iterations), ctypes.byref(ms)))
        del made
        return ms.value

    def close(self):
        if self._h:
            lib().thip_executable_destroy(self._h)
            self._h = ctypes.c_void_p()
