"""Host-side mirror of the TorqHL ops on the quantized path.

A :class:`Program` is the list of ``torq_hl.*`` ops of one dispatch, as they
leave the reference's Linalg->TorqHL conversion
(compiler/torq/Codegen/TORQLowerExecutableTargetPass.cpp:125,142): literal
``pad`` / ``stride``, O,I,KH,KW weights, interleaved ``scale_bias``.  Method
names, keyword names and their meaning are those of the op definitions in
compiler/torq/Dialect/TorqHL/TorqHLOps.td (add :48-69, matmul :85-99, conv2d
:119-143, depthwise_conv2d :145-170, fully_connected :172-190, avg_pool2d
:192-208, transpose :397-407, maxpool2d :435-453).  ``serialize()`` hands the
program to the emitter behind the C-ABI and returns the dispatch descriptor.
"""
import ctypes

import numpy as np

from . import runtime as rt


class Value:
    """A tensor value of a program: a binding, a constant or an intermediate."""

    def __init__(self, program, index, shape, dtype, kind):
        self.program = program
        self.index = index
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        self.kind = kind

    def __repr__(self):
        return "Value(%s #%d %s %s)" % (self.kind, self.index, self.shape, self.dtype)


def _window_out(size, k, p0, p1, stride):
    return (size + p0 + p1 - k) // stride + 1


class Program:
    def __init__(self):
        self._h = ctypes.c_void_p()
        rt.check(rt.lib().thip_program_create(ctypes.byref(self._h)))
        self._keep = []

    def close(self):
        if self._h:
            rt.lib().thip_program_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ---- values -------------------------------------------------------------
    def _dtype_code(self, dtype):
        try:
            return rt._NP_TO_DTYPE[np.dtype(dtype)]
        except KeyError:
            raise rt.ThipError(rt.UNIMPLEMENTED, "element type %s is not supported" % np.dtype(dtype))

    def set_name(self, name):
        """Name of the hal.executable.export the program stands for (dump directories and profile rows carry it)."""
        rt.check(rt.lib().thip_program_set_name(self._h, name.encode()))

    def binding(self, index, shape, dtype=np.int8):
        v = ctypes.c_int32()
        rt.check(rt.lib().thip_program_binding(self._h, int(index), self._dtype_code(dtype), len(shape),
                                               rt._shape_array(shape), ctypes.byref(v)))
        return Value(self, v.value, shape, dtype, "binding")

    def constant(self, array):
        a = np.ascontiguousarray(array)
        shape = a.shape if a.ndim else (1,)
        v = ctypes.c_int32()
        rt.check(rt.lib().thip_program_constant(self._h, self._dtype_code(a.dtype), len(shape),
                                                rt._shape_array(shape), a.ctypes.data_as(ctypes.c_void_p),
                                                a.nbytes, ctypes.byref(v)))
        return Value(self, v.value, shape, a.dtype, "constant")

    def tensor(self, shape, dtype=np.int8):
        v = ctypes.c_int32()
        rt.check(rt.lib().thip_program_tensor(self._h, self._dtype_code(dtype), len(shape),
                                              rt._shape_array(shape), ctypes.byref(v)))
        return Value(self, v.value, shape, dtype, "tensor")

    def view(self, base, shape, offset=0):
        """The same bytes under another shape (tensor.collapse_shape / expand_shape / a contiguous slice): `shape`
        elements of `base` starting `offset` elements into it."""
        v = ctypes.c_int32()
        rt.check(rt.lib().thip_program_view(self._h, base.index, int(offset), len(shape), rt._shape_array(shape),
                                            ctypes.byref(v)))
        return Value(self, v.value, shape, base.dtype, "view")

    def _as_value(self, x):
        if isinstance(x, Value):
            return x
        return self.constant(x)

    def _init_or_new(self, init, shape, dtype):
        if init is None:
            return self.tensor(shape, dtype)
        return init

    # ---- ops ----------------------------------------------------------------
    def conv2d(self, input, weights, scale_bias, *, input_zp, output_zp, output_min, output_max,
               shift_factor, pad, stride, init=None, weight_zp=0, groups=1, dilation=(1, 1),
               vectorization_mode=0, nhwc_input=False, segment_output=False, out_dtype=np.int8):
        weights = self._as_value(weights)
        scale_bias = self._as_value(scale_bias)
        O, _, KH, KW = weights.shape
        if nhwc_input:
            N, H, W, _ = input.shape
        else:
            N, _, H, W = input.shape
        OH = _window_out(H, KH, pad[2], pad[3], stride[0])
        OW = _window_out(W, KW, pad[0], pad[1], stride[1])
        shape = (N, OH, OW, O) if nhwc_input else (N, O, OH, OW)
        if input.dtype == np.uint16:  # bf16 bit patterns in, bf16 out
            out_dtype = np.uint16
        init = self._init_or_new(init, shape, out_dtype)
        op = rt.HlConv2d(init.index, input_zp, weight_zp, output_zp, output_min, output_max, shift_factor,
                         groups, (ctypes.c_int64 * 4)(*pad), (ctypes.c_int64 * 2)(*stride),
                         (ctypes.c_int64 * 2)(*dilation), vectorization_mode, weights.index,
                         scale_bias.index, input.index, int(nhwc_input), int(segment_output))
        rt.check(rt.lib().thip_hl_conv2d(self._h, ctypes.byref(op)))
        return init

    def depthwise_conv2d(self, input, weights, scale_bias, *, input_zp, output_zp, output_min,
                         output_max, shift_factor, pad, stride, init=None, weight_zp=0, groups=None,
                         dilation=(1, 1), vectorization_mode=0, nhwc_input=False,
                         segment_output=False, is_dw1d_stride1=False):
        weights = self._as_value(weights)
        scale_bias = self._as_value(scale_bias)
        C, _, KH, KW = weights.shape
        if nhwc_input:
            N, H, W, _ = input.shape
        else:
            N, _, H, W = input.shape
        OH = _window_out(H, KH, pad[2], pad[3], stride[0])
        OW = _window_out(W, KW, pad[0], pad[1], stride[1])
        shape = (N, OH, OW, C) if nhwc_input else (N, C, OH, OW)
        init = self._init_or_new(init, shape, np.uint16 if input.dtype == np.uint16 else np.int8)
        op = rt.HlDepthwiseConv2d(init.index, input_zp, weight_zp, output_zp, output_min, output_max,
                                  shift_factor, C if groups is None else groups,
                                  (ctypes.c_int64 * 4)(*pad), (ctypes.c_int64 * 2)(*stride),
                                  (ctypes.c_int64 * 2)(*dilation), vectorization_mode, weights.index,
                                  scale_bias.index, input.index, int(nhwc_input), int(segment_output),
                                  int(is_dw1d_stride1))
        rt.check(rt.lib().thip_hl_depthwise_conv2d(self._h, ctypes.byref(op)))
        return init

    def fully_connected(self, input, weights, scale_bias, *, output_zp, output_min, output_max,
                        shift_factor, init=None, input_zp=-128, weight_zp=0, vectorization_mode=0,
                        out_dtype=np.int8):
        weights = self._as_value(weights)
        scale_bias = self._as_value(scale_bias)
        N, K = weights.shape
        M = int(np.prod(input.shape)) // K
        if input.dtype == np.uint16:  # bf16 bit patterns in, bf16 out
            out_dtype = np.uint16
        init = self._init_or_new(init, (M, N), out_dtype)
        op = rt.HlFullyConnected(init.index, input_zp, weight_zp, output_zp, output_min, output_max,
                                 shift_factor, vectorization_mode, weights.index, scale_bias.index,
                                 input.index)
        rt.check(rt.lib().thip_hl_fully_connected(self._h, ctypes.byref(op)))
        return init

    def matmul(self, input1, input2, scale_bias, *, output_zp, output_min, output_max, shift,
               init=None, out_dtype=np.int32):
        input2 = self._as_value(input2)
        scale_bias = self._as_value(scale_bias)
        batch = ()
        if len(input1.shape) == 3 or len(input2.shape) == 3:
            b1 = input1.shape[0] if len(input1.shape) == 3 else 1
            b2 = input2.shape[0] if len(input2.shape) == 3 else 1
            batch = (max(b1, b2),)
        shape = batch + (input1.shape[-2], input2.shape[-1])
        if input1.dtype == np.uint16:  # bf16 bit patterns in, bf16 out
            out_dtype = np.uint16
        init = self._init_or_new(init, shape, out_dtype)
        op = rt.HlMatmul(init.index, output_zp, output_min, output_max, shift, scale_bias.index,
                         input1.index, input2.index)
        rt.check(rt.lib().thip_hl_matmul(self._h, ctypes.byref(op)))
        return init

    def maxpool2d(self, input, *, input_zp, output_min, output_max, stride, pad, kernel, init=None,
                  weights=None, scale_bias=None, segment_output=False, nhwc_input=False):
        if nhwc_input:
            N, H, W, C = input.shape
        else:
            N, C, H, W = input.shape
        OH = _window_out(H, kernel[0], pad[2], pad[3], stride[0])
        OW = _window_out(W, kernel[1], pad[0], pad[1], stride[1])
        shape = (N, OH, OW, C) if nhwc_input else (N, C, OH, OW)
        init = self._init_or_new(init, shape, np.uint16 if input.dtype == np.uint16 else np.int8)
        widx = self._as_value(weights).index if weights is not None else -1
        sidx = self._as_value(scale_bias).index if scale_bias is not None else -1
        op = rt.HlMaxPool2d(init.index, input_zp, output_min, output_max, (ctypes.c_int64 * 2)(*stride),
                            (ctypes.c_int64 * 4)(*pad), (ctypes.c_int64 * 2)(*kernel), widx, sidx,
                            input.index, int(segment_output), int(nhwc_input))
        rt.check(rt.lib().thip_hl_maxpool2d(self._h, ctypes.byref(op)))
        return init

    def avg_pool2d(self, input, weights, scale_bias, *, input_zp, output_zp, output_min, output_max,
                   shift_factor, init=None):
        weights = self._as_value(weights)
        scale_bias = self._as_value(scale_bias)
        N, _, _, C = input.shape
        init = self._init_or_new(init, (N, 1, 1, C), np.uint16 if input.dtype == np.uint16 else np.int8)
        op = rt.HlAvgPool2d(init.index, input_zp, output_zp, output_min, output_max, shift_factor,
                            weights.index, scale_bias.index, input.index)
        rt.check(rt.lib().thip_hl_avg_pool2d(self._h, ctypes.byref(op)))
        return init

    def add(self, input1, input2, weights, scale_bias, *, output_zp, output_min, output_max,
            shift_factor, init=None, name="add", input_zp=0, segment_output=False,
            rhs_is_scalar=False):
        weights = self._as_value(weights)
        scale_bias = self._as_value(scale_bias)
        init = self._init_or_new(init, input1.shape, input1.dtype)
        op = rt.HlAdd(init.index, name.encode(), input_zp, output_zp, output_min, output_max,
                      shift_factor, weights.index, scale_bias.index, input1.index, input2.index,
                      int(segment_output), int(rhs_is_scalar))
        rt.check(rt.lib().thip_hl_add(self._h, ctypes.byref(op)))
        return init

    def expand_weights(self, input, scale, scale_bias, *, block_size, output_min, output_max, init=None):
        """torq_hl.expand_weights: int8 weights K,N times per-block bf16 scales plus float biases -> bf16 1,K,N."""
        input = self._as_value(input)
        scale = self._as_value(scale)
        scale_bias = self._as_value(scale_bias)
        K, N = input.shape
        init = self._init_or_new(init, (1, K, N), np.uint16)
        op = rt.HlExpandWeights(init.index, scale_bias.index, output_min, output_max, scale.index, input.index,
                                block_size)
        rt.check(rt.lib().thip_hl_expand_weights(self._h, ctypes.byref(op)))
        return init

    def fma(self, input, weights, scale_bias, *, output_zp, output_min, output_max, shift_factor, init=None,
            out_dtype=np.int8):
        """torq_hl.fma, the stand-alone rescale: init = R1(input * weights[0])."""
        weights = self._as_value(weights)
        scale_bias = self._as_value(scale_bias)
        init = self._init_or_new(init, input.shape, out_dtype)
        op = rt.HlFma(init.index, output_zp, output_min, output_max, shift_factor, weights.index, scale_bias.index,
                      input.index)
        rt.check(rt.lib().thip_hl_fma(self._h, ctypes.byref(op)))
        return init

    def mul(self, input1, input2, scale_bias, *, output_zp, output_min, output_max, shift, init=None,
            out_dtype=np.int8):
        """torq_hl.mul: init = R1(input1 * input2); an input of one element is broadcast."""
        input1 = self._as_value(input1)
        input2 = self._as_value(input2)
        scale_bias = self._as_value(scale_bias)
        shape = input1.shape if int(np.prod(input1.shape)) >= int(np.prod(input2.shape)) else input2.shape
        init = self._init_or_new(init, shape, out_dtype)
        op = rt.HlMul(init.index, output_zp, output_min, output_max, scale_bias.index, shift, input1.index,
                      input2.index)
        rt.check(rt.lib().thip_hl_mul(self._h, ctypes.byref(op)))
        return init

    def act(self, input, name, *, min_int=0, max_int=0, min_fp=0.0, max_fp=0.0, input_zp=0, output_zp=0, init=None,
            out_dtype=None, weights=None):
        """torq_hl.act on integers: name in clamp / abs / negate / i2i."""
        init = self._init_or_new(init, input.shape, input.dtype if out_dtype is None else out_dtype)
        w = rt.NO_VALUE if weights is None else self._as_value(weights).index
        op = rt.HlAct(init.index, name.encode(), input_zp, output_zp, int(min_int), int(max_int), min_fp, max_fp,
                      input.index, w)
        rt.check(rt.lib().thip_hl_act(self._h, ctypes.byref(op)))
        return init

    def elementwiseunary(self, op_type, input, *, init=None):
        """torq_hl.elementwiseunary: op_type 3 BITWISE_NOT (integers) or 12 LOGICAL_NOT (i1, carried as uint8 0 / 1)."""
        init = self._init_or_new(init, input.shape, input.dtype)
        op = rt.HlElementwiseUnary(init.index, int(op_type), input.index)
        rt.check(rt.lib().thip_hl_elementwiseunary(self._h, ctypes.byref(op)))
        return init

    def table(self, input, scale_bias, *, dynamic_table=None, static_table=None, init=None, out_dtype=None):
        """torq_hl.table: 256 int32 segment words, either as a constant tensor (dynamic_table) or as the static_table
        attribute; scale_bias = [-128, 128] (the plain lookup)."""
        init = self._init_or_new(init, input.shape, input.dtype if out_dtype is None else out_dtype)
        sb = self._as_value(np.asarray(scale_bias, dtype=np.int32))
        dyn = rt.NO_VALUE if dynamic_table is None else self._as_value(np.asarray(dynamic_table, dtype=np.int32)).index
        if static_table is None:
            words, count = None, 0
        else:
            arr = np.ascontiguousarray(static_table, dtype=np.int32)
            words, count = arr.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), int(arr.size)
        op = rt.HlTable(init.index, sb.index, input.index, dyn, words, count)
        rt.check(rt.lib().thip_hl_table(self._h, ctypes.byref(op)))
        return init

    def elementwiseshift(self, op_type, input1, input2, *, round=False, init=None):
        """torq_hl.elementwiseshift: op_type 0 LSR, 1 LSL, 2 ASR; input2 holds the per-element counts."""
        input2 = self._as_value(input2)
        init = self._init_or_new(init, input1.shape, input1.dtype)
        op = rt.HlElementwiseShift(init.index, int(op_type), int(bool(round)), input1.index, input2.index)
        rt.check(rt.lib().thip_hl_elementwiseshift(self._h, ctypes.byref(op)))
        return init

    def elementwisebinary(self, op_type, input1, input2, *, is_unsigned=False, init=None):
        """torq_hl.elementwisebinary: op_type is the reference's ElementwiseOpEnum value: 0 and, 1 or, 2 xor, 4 minimum,
        5 maximum (result of the inputs' type); 6 greater, 7 greater-equal, 8 equal, 9..11 logical and / or / xor (an i1
        result, carried as uint8 0 / 1)."""
        input2 = self._as_value(input2)
        init = self._init_or_new(init, input1.shape, np.uint8 if int(op_type) >= 6 else input1.dtype)
        op = rt.HlElementwiseBinary(init.index, int(op_type), input1.index, input2.index, int(bool(is_unsigned)))
        rt.check(rt.lib().thip_hl_elementwisebinary(self._h, ctypes.byref(op)))
        return init

    def transpose(self, input, perm, init=None):
        shape = tuple(input.shape[p] for p in perm)
        init = self._init_or_new(init, shape, input.dtype)
        p4 = list(perm) + [0] * (4 - len(perm))
        op = rt.HlTranspose(init.index, len(perm), (ctypes.c_int64 * 4)(*p4), input.index)
        rt.check(rt.lib().thip_hl_transpose(self._h, ctypes.byref(op)))
        return init

    # ---- serialisation ------------------------------------------------------
    def serialize(self):
        """Returns the dispatch descriptor as ``bytes``."""
        blob = ctypes.c_void_p()
        size = ctypes.c_size_t()
        rt.check(rt.lib().thip_program_serialize(self._h, ctypes.byref(blob), ctypes.byref(size)))
        try:
            return ctypes.string_at(blob, size.value)
        finally:
            rt.lib().thip_blob_free(blob)
