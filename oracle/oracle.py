"""numpy front-end of the C oracle (``libtorq_oracle.so``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by the smoke check and by the
benchmark's CPU-baseline leg, never by the product package.  Every function is a
thin ctypes call into ``torq_oracle.c``; argument names follow the TorqHL op
definitions (compiler/torq/Dialect/TorqHL/TorqHLOps.td:48-208,435-453).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libtorq_oracle.so")

NCHW, NHWC = 0, 1


class Requant(ctypes.Structure):
    _fields_ = [
        ("shift", ctypes.c_int32),
        ("output_zp", ctypes.c_int32),
        ("output_min", ctypes.c_int32),
        ("output_max", ctypes.c_int32),
    ]


def build():
    """Compile the oracle with the Makefile next to this file."""
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.torq_act_rescale_clamp.restype = ctypes.c_int64
        L.torq_act_rescale_clamp.argtypes = [ctypes.c_int32] * 3 + [ctypes.POINTER(Requant)]
        L.torq_derive_scale_bias.restype = ctypes.c_int32
        L.torq_oracle_threads.restype = ctypes.c_int
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _i64x(vals):
    return (ctypes.c_int64 * len(vals))(*[int(v) for v in vals])


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


_OUT_DTYPES = {1: np.int8, 2: np.int16, 4: np.int32}


def threads():
    return lib().torq_oracle_threads()


def set_threads(n):
    lib().torq_oracle_set_threads(int(n))


def act_rescale_clamp(acc, bias, scale, shift, output_zp, output_min, output_max):
    rq = Requant(shift, output_zp, output_min, output_max)
    return int(lib().torq_act_rescale_clamp(int(acc), int(bias), int(scale), ctypes.byref(rq)))


def _out_hw(H, W, KH, KW, pad, stride):
    pl, pr, pt, pb = [int(p) for p in pad]
    OH = (H + pt + pb - KH) // int(stride[0]) + 1
    OW = (W + pl + pr - KW) // int(stride[1]) + 1
    return OH, OW


def conv2d(input, weights, scale_bias, *, input_zp, output_zp, output_min, output_max,
           shift_factor, pad, stride, layout=NCHW, out_dtype=np.int8):
    """torq_hl.conv2d; input N,C,H,W (or N,H,W,C when layout=NHWC), weights O,I,KH,KW."""
    x = _c(input, np.int8)
    w = _c(weights, np.int8)
    sb = _c(scale_bias, np.int32)
    if layout == NHWC:
        N, H, W, C = x.shape
    else:
        N, C, H, W = x.shape
    O, I, KH, KW = w.shape
    assert I == C and sb.size == 2 * O
    OH, OW = _out_hw(H, W, KH, KW, pad, stride)
    shape = (N, OH, OW, O) if layout == NHWC else (N, O, OH, OW)
    out = np.empty(shape, dtype=out_dtype)
    rq = Requant(shift_factor, output_zp, output_min, output_max)
    rc = lib().torq_conv2d(_p(x), _p(w), _p(sb), _p(out), N, C, H, W, O, KH, KW, _i64x(pad),
                           _i64x(stride), ctypes.c_int32(input_zp), ctypes.byref(rq), layout,
                           out.itemsize)
    assert rc == 0
    return out


def depthwise_conv2d(input, weights, scale_bias, *, input_zp, output_zp, output_min, output_max,
                     shift_factor, pad, stride, layout=NCHW, out_dtype=np.int8):
    """torq_hl.depthwise_conv2d; weights C,1,KH,KW."""
    x = _c(input, np.int8)
    w = _c(weights, np.int8)
    sb = _c(scale_bias, np.int32)
    if layout == NHWC:
        N, H, W, C = x.shape
    else:
        N, C, H, W = x.shape
    Cw, one, KH, KW = w.shape
    assert Cw == C and one == 1 and sb.size == 2 * C
    OH, OW = _out_hw(H, W, KH, KW, pad, stride)
    shape = (N, OH, OW, C) if layout == NHWC else (N, C, OH, OW)
    out = np.empty(shape, dtype=out_dtype)
    rq = Requant(shift_factor, output_zp, output_min, output_max)
    rc = lib().torq_depthwise_conv2d(_p(x), _p(w), _p(sb), _p(out), N, C, H, W, KH, KW,
                                     _i64x(pad), _i64x(stride), ctypes.c_int32(input_zp),
                                     ctypes.byref(rq), layout, out.itemsize)
    assert rc == 0
    return out


def fully_connected(input, weights, scale_bias, *, output_zp, output_min, output_max,
                    shift_factor, out_dtype=np.int8):
    """torq_hl.fully_connected; input M,K, weights N,K."""
    x = _c(input, np.int8)
    w = _c(weights, np.int8)
    sb = _c(scale_bias, np.int32)
    M, K = x.shape
    N, K2 = w.shape
    assert K == K2 and sb.size == 2 * N
    out = np.empty((M, N), dtype=out_dtype)
    rq = Requant(shift_factor, output_zp, output_min, output_max)
    rc = lib().torq_fully_connected(_p(x), _p(w), _p(sb), _p(out), M, K, N, ctypes.byref(rq),
                                    out.itemsize)
    assert rc == 0
    return out


def matmul(input1, input2, scale_bias, *, output_zp, output_min, output_max, shift,
           out_dtype=np.int32):
    """torq_hl.matmul; input1 [B,]M,K  input2 [B,]K,N; one (bias, scale) pair."""
    a = _c(input1, np.int8)
    b = _c(input2, np.int8)
    sb = _c(scale_bias, np.int32)
    a3 = a.reshape((-1,) + a.shape[-2:]) if a.ndim >= 2 else a.reshape(1, 1, -1)
    b3 = b.reshape((-1,) + b.shape[-2:])
    B = max(a3.shape[0], b3.shape[0])
    _, M, K = a3.shape
    _, K2, N = b3.shape
    assert K == K2 and sb.size >= 2
    out = np.empty((B, M, N), dtype=out_dtype)
    rq = Requant(shift, output_zp, output_min, output_max)
    rc = lib().torq_matmul(_p(a3), _p(b3), _p(sb), _p(out), B, M, K, N,
                           int(a3.shape[0] == 1 and B > 1), int(b3.shape[0] == 1 and B > 1),
                           ctypes.byref(rq), out.itemsize)
    assert rc == 0
    return out


NO_CLAMP_MIN, NO_CLAMP_MAX = -8388608, 0x7f800000  # float bit patterns of -inf / +inf as int32 attributes


def to_bf16(values):
    """float32 array -> bfloat16 bit patterns (uint16), round to nearest even."""
    f = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty(f.shape, dtype=np.uint16)
    flat_in, flat_out = f.reshape(-1), out.reshape(-1)
    u = flat_in.view(np.uint32).astype(np.uint64)
    r = ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = (u & 0x7fffffff) > 0x7f800000
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    flat_out[:] = r
    return out


def from_bf16(bits):
    """bfloat16 bit patterns (uint16) -> float32."""
    b = np.ascontiguousarray(bits, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32)


def fully_connected_bf16(input, weights, bias, *, output_min=NO_CLAMP_MIN, output_max=NO_CLAMP_MAX):
    """torq_hl.fully_connected on bf16 bit patterns; input M,K, weights N,K, bias N float32."""
    x = _c(input, np.uint16)
    w = _c(weights, np.uint16)
    b = _c(bias, np.float32)
    M, K = x.shape
    N, K2 = w.shape
    assert K == K2 and b.size == N
    out = np.empty((M, N), dtype=np.uint16)
    rc = lib().torq_fully_connected_bf16(_p(x), _p(w), _p(b), _p(out), M, K, N, int(output_min), int(output_max))
    assert rc == 0
    return out


def matmul_bf16(input1, input2, bias, *, output_min=NO_CLAMP_MIN, output_max=NO_CLAMP_MAX):
    """torq_hl.matmul on bf16 bit patterns; input1 [B,]M,K  input2 [B,]K,N; one float32 bias."""
    a = _c(input1, np.uint16)
    b = _c(input2, np.uint16)
    bias = _c(bias, np.float32)
    a3 = a.reshape((-1,) + a.shape[-2:])
    b3 = b.reshape((-1,) + b.shape[-2:])
    B = max(a3.shape[0], b3.shape[0])
    _, M, K = a3.shape
    _, K2, N = b3.shape
    assert K == K2 and bias.size >= 1
    out = np.empty((B, M, N), dtype=np.uint16)
    rc = lib().torq_matmul_bf16(_p(a3), _p(b3), _p(bias), _p(out), B, M, K, N, int(a3.shape[0] == 1 and B > 1),
                                int(b3.shape[0] == 1 and B > 1), int(output_min), int(output_max))
    assert rc == 0
    return out


def conv2d_bf16(input, weights, bias, *, pad, stride, output_min=NO_CLAMP_MIN, output_max=NO_CLAMP_MAX, layout=NCHW):
    """torq_hl.conv2d on bf16 bit patterns; weights O,I,KH,KW; bias O float32; zero padding."""
    x = _c(input, np.uint16)
    w = _c(weights, np.uint16)
    b = _c(bias, np.float32)
    if layout == NHWC:
        N, H, W, C = x.shape
    else:
        N, C, H, W = x.shape
    O, I, KH, KW = w.shape
    assert I == C and b.size == O
    OH, OW = _out_hw(H, W, KH, KW, pad, stride)
    out = np.empty((N, OH, OW, O) if layout == NHWC else (N, O, OH, OW), dtype=np.uint16)
    rc = lib().torq_conv2d_bf16(_p(x), _p(w), _p(b), _p(out), N, C, H, W, O, KH, KW, _i64x(pad), _i64x(stride),
                                int(output_min), int(output_max), layout)
    assert rc == 0
    return out


def depthwise_conv2d_bf16(input, weights, bias, *, pad, stride, output_min=NO_CLAMP_MIN, output_max=NO_CLAMP_MAX, layout=NCHW):
    """torq_hl.depthwise_conv2d on bf16 bit patterns; weights C,1,KH,KW; bias C float32."""
    x = _c(input, np.uint16)
    w = _c(weights, np.uint16)
    b = _c(bias, np.float32)
    if layout == NHWC:
        N, H, W, C = x.shape
    else:
        N, C, H, W = x.shape
    C2, one, KH, KW = w.shape
    assert C2 == C and one == 1 and b.size == C
    OH, OW = _out_hw(H, W, KH, KW, pad, stride)
    out = np.empty((N, OH, OW, C) if layout == NHWC else (N, C, OH, OW), dtype=np.uint16)
    rc = lib().torq_depthwise_conv2d_bf16(_p(x), _p(w), _p(b), _p(out), N, C, H, W, KH, KW, _i64x(pad), _i64x(stride),
                                          int(output_min), int(output_max), layout)
    assert rc == 0
    return out


def add_bf16(input1, input2, weights, bias, *, output_min=NO_CLAMP_MIN, output_max=NO_CLAMP_MAX):
    """torq_hl.add on bf16 bit patterns: two bf16 weights, one float32 bias."""
    a = _c(input1, np.uint16)
    b = _c(input2, np.uint16)
    assert a.shape == b.shape
    w = _c(weights, np.uint16)
    bias = _c(bias, np.float32)
    assert w.size >= 2 and bias.size >= 1
    out = np.empty(a.shape, dtype=np.uint16)
    rc = lib().torq_add_bf16(_p(a), _p(b), _p(w), _p(bias), _p(out), ctypes.c_size_t(a.size), int(output_min), int(output_max))
    assert rc == 0
    return out


def avg_pool2d_bf16(input, weight, bias, *, output_min=NO_CLAMP_MIN, output_max=NO_CLAMP_MAX):
    """torq_hl.avg_pool2d on bf16 bit patterns (N,H,W,C): one bf16 weight, one float32 bias; result N,1,1,C."""
    x = _c(input, np.uint16)
    N, H, W, C = x.shape
    w = _c(weight, np.uint16).reshape(-1)
    bias = _c(bias, np.float32).reshape(-1)
    assert w.size >= 1 and bias.size >= 1
    out = np.empty((N, 1, 1, C), dtype=np.uint16)
    rc = lib().torq_avg_pool2d_bf16(_p(x), ctypes.c_uint16(int(w[0])), _p(bias), _p(out), N, H, W, C, int(output_min), int(output_max))
    assert rc == 0
    return out


def expand_weights(weights, scale, bias, *, block_size, output_min=NO_CLAMP_MIN, output_max=NO_CLAMP_MAX):
    """torq_hl.expand_weights: int8 weights [K, N], bf16 scales [K / block_size, N], float32 biases
    [K / block_size, >= N]; result bf16 bit patterns [K, N]."""
    w = _c(weights, np.int8)
    K, N = w.shape
    sc = _c(scale, np.uint16)
    b = _c(bias, np.float32)
    G = K // block_size
    assert G * block_size == K and sc.shape == (G, N) and b.shape[0] == G and b.shape[1] >= N
    out = np.empty((K, N), dtype=np.uint16)
    rc = lib().torq_expand_weights(_p(w), _p(sc), _p(b), _p(out), K, N, int(block_size), int(b.shape[1]), int(output_min), int(output_max))
    assert rc == 0
    return out


def maxpool2d(input, *, input_zp, output_min, output_max, stride, pad, kernel, layout=NCHW):
    """torq_hl.maxpool2d."""
    x = _c(input, np.int8)
    if layout == NHWC:
        N, H, W, C = x.shape
    else:
        N, C, H, W = x.shape
    KH, KW = int(kernel[0]), int(kernel[1])
    OH, OW = _out_hw(H, W, KH, KW, pad, stride)
    shape = (N, OH, OW, C) if layout == NHWC else (N, C, OH, OW)
    out = np.empty(shape, dtype=np.int8)
    rc = lib().torq_maxpool2d(_p(x), _p(out), N, C, H, W, KH, KW, _i64x(pad), _i64x(stride),
                              ctypes.c_int32(input_zp), ctypes.c_int32(output_min),
                              ctypes.c_int32(output_max), layout)
    assert rc == 0
    return out


def avg_pool2d(input, scale_bias, *, output_zp, output_min, output_max, shift_factor, weight=1):
    """torq_hl.avg_pool2d (global); input N,H,W,C -> N,1,1,C."""
    x = _c(input, np.int8)
    sb = _c(scale_bias, np.int32)
    N, H, W, C = x.shape
    out = np.empty((N, 1, 1, C), dtype=np.int8)
    rq = Requant(shift_factor, output_zp, output_min, output_max)
    rc = lib().torq_avg_pool2d(_p(x), ctypes.c_int8(weight), _p(sb), _p(out), N, H, W, C,
                               ctypes.byref(rq))
    assert rc == 0
    return out


def add(input1, input2, weights, scale_bias, *, output_zp, output_min, output_max, shift_factor):
    """torq_hl.add (tensor + tensor)."""
    a = _c(input1, np.int8)
    b = _c(input2, np.int8)
    assert a.shape == b.shape
    w = _c(weights, np.int16)
    sb = _c(scale_bias, np.int32)
    out = np.empty(a.shape, dtype=np.int8)
    rq = Requant(shift_factor, output_zp, output_min, output_max)
    rc = lib().torq_add(_p(a), _p(b), _p(w), _p(sb), _p(out), ctypes.c_size_t(a.size),
                        ctypes.byref(rq))
    assert rc == 0
    return out


_INT_TYPES = (np.int8, np.int16, np.int32)
ACT_MODES = {"clamp": 0, "abs": 1, "negate": 2, "i2i": 3}


def _int_array(a, truth_values=False):
    """int8 / int16 / int32 data; with truth_values also uint8 arrays of 0 / 1 (i1 tensors, one byte per element)."""
    a = np.ascontiguousarray(a)
    if truth_values and a.dtype == np.uint8:
        assert a.size == 0 or int(a.max()) <= 1, "an i1 tensor holds 0 or 1"
        return a
    assert a.dtype in [np.dtype(t) for t in _INT_TYPES], a.dtype
    return a


def fma(input, weights, scale_bias, *, output_zp, output_min, output_max, shift_factor, out_dtype=np.int8):
    """torq_hl.fma (stand-alone rescale): one scalar weight, one [bias, scale] pair."""
    x = _int_array(input)
    w = np.asarray(weights).reshape(-1)
    sb = _c(scale_bias, np.int32)
    out = np.empty(x.shape, dtype=out_dtype)
    rq = Requant(shift_factor, output_zp, output_min, output_max)
    rc = lib().torq_fma(_p(x), x.itemsize, ctypes.c_int32(int(w[0])), _p(sb), _p(out), out.itemsize, ctypes.c_size_t(x.size), ctypes.byref(rq))
    assert rc == 0
    return out


def mul(input1, input2, scale_bias, *, output_zp, output_min, output_max, shift, out_dtype=np.int8):
    """torq_hl.mul: elementwise product (a one-element input is broadcast), one [bias, scale] pair."""
    a = _int_array(input1)
    b = _int_array(input2)
    assert a.dtype == b.dtype
    shape = a.shape if a.size >= b.size else b.shape
    count = max(a.size, b.size)
    sb = _c(scale_bias, np.int32)
    out = np.empty(shape, dtype=out_dtype)
    rq = Requant(shift, output_zp, output_min, output_max)
    rc = lib().torq_mul(_p(a), ctypes.c_size_t(a.size), _p(b), ctypes.c_size_t(b.size), a.itemsize, _p(sb), _p(out), out.itemsize,
                        ctypes.c_size_t(count), ctypes.byref(rq))
    assert rc == 0
    return out


def act(input, name, *, min_int=0, max_int=0, out_dtype=None):
    """torq_hl.act on integers: name in clamp / abs / negate / i2i."""
    x = _int_array(input)
    out = np.empty(x.shape, dtype=x.dtype if out_dtype is None else out_dtype)
    rc = lib().torq_act(_p(x), x.itemsize, _p(out), out.itemsize, ctypes.c_size_t(x.size), ACT_MODES[name], ctypes.c_int64(int(min_int)),
                        ctypes.c_int64(int(max_int)))
    assert rc == 0
    return out


BINARY_MODES = {"and": 0, "or": 1, "xor": 2, "minimum": 4, "maximum": 5}


def elementwise_binary(op_type, input1, input2, *, is_unsigned=False):
    """torq_hl.elementwisebinary: and / or / xor / minimum / maximum on two integer tensors of one type."""
    a = _int_array(input1)
    b = _int_array(input2)
    assert a.dtype == b.dtype and a.shape == b.shape
    out = np.empty(a.shape, dtype=a.dtype)
    rc = lib().torq_elementwise_binary(BINARY_MODES[op_type], _p(a), _p(b), a.itemsize, int(bool(is_unsigned)), _p(out), ctypes.c_size_t(a.size))
    assert rc == 0
    return out


def elementwise_compare(op_type, input1, input2, *, is_unsigned=False):
    """torq_hl.elementwisebinary, comparison / logical modes (the enum's values 6..11): an i1 result as uint8 0 / 1."""
    a = _int_array(input1, truth_values=True)
    b = _int_array(input2, truth_values=True)
    assert a.dtype == b.dtype and a.shape == b.shape
    out = np.empty(a.shape, dtype=np.uint8)
    rc = lib().torq_elementwise_compare(int(op_type), _p(a), _p(b), a.itemsize, int(bool(is_unsigned)), _p(out), ctypes.c_size_t(a.size))
    assert rc == 0
    return out


def elementwise_unary(op_type, input):
    """torq_hl.elementwiseunary: 3 bitwise not, 12 logical not (on i1 bytes)."""
    a = _int_array(input, truth_values=True)
    out = np.empty(a.shape, dtype=a.dtype)
    rc = lib().torq_elementwise_unary(int(op_type), _p(a), a.itemsize, _p(out), ctypes.c_size_t(a.size))
    assert rc == 0
    return out


def elementwise_shift(op_type, input1, input2, *, round=False):
    """torq_hl.elementwiseshift: 0 logical right, 1 logical left, 2 arithmetic right; counts per element in input2."""
    a = _int_array(input1)
    b = _int_array(input2)
    assert a.dtype == b.dtype and a.shape == b.shape
    out = np.empty(a.shape, dtype=a.dtype)
    rc = lib().torq_elementwise_shift(int(op_type), int(bool(round)), _p(a), _p(b), a.itemsize, _p(out), ctypes.c_size_t(a.size))
    assert rc == 0
    return out


def table(input, words, out_dtype, *, bias=-128, scale=128):
    """torq_hl.table with segment words `words` (int32): the plain lookup the extract patterns produce."""
    x = _int_array(input)
    assert x.dtype in (np.int8, np.int16)
    w = _c(words, np.int32)
    out = np.empty(x.shape, dtype=out_dtype)
    rc = lib().torq_table(_p(x), x.itemsize, _p(w), int(w.size), int(bias), int(scale), _p(out), out.itemsize, ctypes.c_size_t(x.size))
    if rc != 0:
        raise ValueError("torq_table: an input needs an interpolated or out-of-table entry, which the oracle does not define")
    return out


def per_channel_sum(weights):
    w = _c(weights, np.int8)
    ch = w.shape[0]
    sums = np.empty(ch, dtype=np.int64)
    lib().torq_per_channel_sum(_p(w), ch, int(w.size // ch), _p(sums))
    return sums


def derive_scale_bias(multiplier, shift, tosa_bias, weight_sum, input_zp):
    """R2: returns (scale_bias int32[2*channels], shift_factor)."""
    m = _c(multiplier, np.int32)
    s = _c(shift, np.int8)
    ch = m.size
    tb = _c(tosa_bias, np.int32) if tosa_bias is not None else None
    ws = _c(weight_sum, np.int64) if weight_sum is not None else None
    sb = np.empty(2 * ch, dtype=np.int32)
    sf = lib().torq_derive_scale_bias(_p(m), _p(s), _p(tb) if tb is not None else None,
                                      _p(ws) if ws is not None else None,
                                      ctypes.c_int32(input_zp), ch, _p(sb))
    return sb, int(sf)


def derive_add_params(m0, m1, zp0, zp1, sign=1):
    """Returns (weights int16[2], scale_bias int32[2], shift_factor) or None if rejected."""
    w = np.empty(2, dtype=np.int16)
    sb = np.empty(2, dtype=np.int32)
    sf = ctypes.c_int32(0)
    rc = lib().torq_derive_add_params(ctypes.c_double(m0), ctypes.c_double(m1),
                                      ctypes.c_int32(zp0), ctypes.c_int32(zp1), int(sign),
                                      _p(w), _p(sb), ctypes.byref(sf))
    if rc != 0:
        return None
    return w, sb, sf.value


def derive_avgpool_params(H, W, input_zp):
    sb = np.empty(2, dtype=np.int32)
    sf = ctypes.c_int32(0)
    lib().torq_derive_avgpool_params(int(H), int(W), ctypes.c_int32(input_zp), _p(sb),
                                     ctypes.byref(sf))
    return sb, sf.value
