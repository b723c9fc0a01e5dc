"""Seeded synthetic workloads at the benchmark shapes.

Each builder returns a :class:`Workload`: the TorqHL program (one or more ops),
the host input arrays in binding order, the output shapes, and the algorithmic
work (ops and bytes) used for roofline accounting.

Requantisation parameters are derived the way the reference's patterns derive
them (compile side, unchanged by this backend):
  shift_factor = min_c shift[c]           compiler/torq/Conversions/LinalgToTorqHL/PatternUtils.cpp:3230-3283
  scale[c] = multiplier[c] >> (shift[c] - shift_factor)                   PatternUtils.cpp:3536-3548
  bias[c]  = tosa_bias[c] - input_zp * sum(w[c])        compiler/torq/Utils/ConversionUtils.h:301-329
  scale_bias = interleave(bias, scale)                 compiler/torq/Utils/ConversionUtils.cpp:88-103
"""
import numpy as np

from .torq_hl import Program


class Workload:
    def __init__(self, name, program, inputs, outputs, ops, bytes_, attrs=None):
        self.name = name
        self.program = program
        self.inputs = inputs      # list of numpy arrays, binding 0..n-1
        self.outputs = outputs    # list of (shape, dtype), bindings n..
        self.ops = ops            # algorithmic integer ops (1 MAC = 2 ops)
        self.bytes = bytes_       # algorithmic bytes: every operand once + output once
        self.attrs = attrs or {}  # the op parameters, for the checker


def derive_scale_bias(multiplier, shift, tosa_bias, weights, input_zp):
    """R2 for conv / depthwise / fully_connected.  weights: [channels, ...]."""
    multiplier = np.asarray(multiplier, dtype=np.int32)
    shift = np.asarray(shift, dtype=np.int64)
    shift_factor = int(shift.min())
    scale = (multiplier.astype(np.int64) >> (shift - shift_factor)).astype(np.int32)
    wsum = weights.reshape(weights.shape[0], -1).astype(np.int64).sum(axis=1)
    bias = (np.asarray(tosa_bias, dtype=np.int64) - wsum * int(input_zp)).astype(np.int32)
    sb = np.empty(2 * multiplier.size, dtype=np.int32)
    sb[0::2] = bias
    sb[1::2] = scale
    return sb, shift_factor


def random_requant(rng, channels, realistic):
    """Per-channel TOSA (multiplier, shift).  The literal benchmark ranges (shift 6..12)
    saturate every output; `realistic` draws shifts 36..42 so the rounding path is exercised."""
    mult = rng.integers(1 << 30, (1 << 31) - 1, size=channels, endpoint=True, dtype=np.int64).astype(np.int32)
    if realistic:
        shift = rng.integers(36, 42, size=channels, endpoint=True)
    else:
        shift = rng.integers(6, 12, size=channels, endpoint=True)
    return mult, shift.astype(np.int8)


def conv2d_workload(N=1, H=112, W=112, C=32, O=64, KH=3, KW=3, stride=(1, 1), pad=(1, 1, 1, 1),
                    input_zp=-3, output_zp=5, output_min=5, output_max=127, realistic=False,
                    nhwc=True, seed=1000):
    """benchmark configuration 0 by default: NHWC 1x112x112x32 -> 1x112x112x64, 3x3, SAME."""
    rng = np.random.default_rng(seed)
    x = rng.integers(-128, 127, size=(N, H, W, C), endpoint=True, dtype=np.int8)
    w_hwio = rng.integers(-127, 127, size=(KH, KW, C, O), endpoint=True, dtype=np.int8)
    w = np.ascontiguousarray(w_hwio.transpose(3, 2, 0, 1))  # O,I,KH,KW as the op takes them
    tosa_bias = rng.integers(-(1 << 15), 1 << 15, size=O, endpoint=True, dtype=np.int64)
    mult, shift = random_requant(rng, O, realistic)
    sb, sf = derive_scale_bias(mult, shift, tosa_bias, w, input_zp)
    attrs = dict(input_zp=input_zp, output_zp=output_zp, output_min=output_min, output_max=output_max,
                 shift_factor=sf, pad=tuple(pad), stride=tuple(stride))
    p = Program()
    if not nhwc:
        x = np.ascontiguousarray(x.transpose(0, 3, 1, 2))
    inp = p.binding(0, x.shape)
    OH = (H + pad[2] + pad[3] - KH) // stride[0] + 1
    OW = (W + pad[0] + pad[1] - KW) // stride[1] + 1
    oshape = (N, OH, OW, O) if nhwc else (N, O, OH, OW)
    out = p.binding(1, oshape)
    p.conv2d(inp, w, sb, init=out, nhwc_input=nhwc, **attrs)
    macs = N * OH * OW * O * KH * KW * C
    bytes_ = x.nbytes + w.nbytes + sb.nbytes + N * OH * OW * O
    attrs.update(weights=w, scale_bias=sb, nhwc=nhwc)
    return Workload("conv2d_%dx%dx%dx%d_o%d_k%dx%d" % (N, H, W, C, O, KH, KW), p, [x], [(oshape, np.int8)],
                    2 * macs, bytes_, attrs)


def fully_connected_workload(M, K, N, realistic=False, output_zp=5, output_min=-128, output_max=127,
                             seed=1001, shift=None, zeros=False):
    """benchmark configuration 1: int8 [M,K] x [N,K]^T with per-column requant.

    `shift` forces one shift_factor for every column (multipliers drawn so that outputs still spread).
    `zeros`: both operands all zero (the same work on data that toggles nothing: a power calibration)."""
    rng = np.random.default_rng(seed)
    x = rng.integers(-128, 127, size=(M, K), endpoint=True, dtype=np.int8)
    w = rng.integers(-128, 127, size=(N, K), endpoint=True, dtype=np.int8)
    if zeros:
        x[...] = 0
        w[...] = 0
    tosa_bias = rng.integers(-(1 << 15), 1 << 15, size=N, endpoint=True, dtype=np.int64)
    if shift is None:
        mult, shift = random_requant(rng, N, realistic)
    else:
        top = min(max(int(shift) - 14, 1), 31)
        mult = rng.integers(1 << (top - 1), (1 << top) - 1, size=N, endpoint=True, dtype=np.int64).astype(np.int32)
        shift = np.full(N, int(shift), dtype=np.int8)
    sb, sf = derive_scale_bias(mult, shift, tosa_bias, w, 0)
    attrs = dict(output_zp=output_zp, output_min=output_min, output_max=output_max, shift_factor=sf)
    p = Program()
    inp = p.binding(0, (M, K))
    out = p.binding(1, (M, N))
    p.fully_connected(inp, w, sb, init=out, **attrs)
    bytes_ = x.nbytes + w.nbytes + sb.nbytes + M * N
    attrs.update(weights=w, scale_bias=sb)
    return Workload("fully_connected_%dx%dx%d" % (M, K, N), p, [x], [((M, N), np.int8)], 2 * M * K * N,
                    bytes_, attrs)


def matmul_workload(B, M, K, N, batch1=True, batch2=True, constant_rhs=False, out_dtype=np.int16, bias=0, scale=1, shift=0,
                    output_zp=0, clamp=None, seed=1022):
    """int8 torq_hl.matmul [B,]M,K x [B,]K,N with ONE (bias, scale) pair and an int8 / int16 / int32 result; input2 is a
    run-time binding unless constant_rhs.  The defaults are what the matmul patterns produce (bias 0, scale 1, shift 0,
    the clamp = the range of the result type; compiler/torq/Conversions/LinalgToTorqHL/MatmulPattern.cpp:925-994)."""
    rng = np.random.default_rng(seed)
    a = rng.integers(-128, 127, size=(B, M, K) if batch1 else (M, K), endpoint=True, dtype=np.int8)
    b = rng.integers(-128, 127, size=(B, K, N) if batch2 else (K, N), endpoint=True, dtype=np.int8)
    sb = np.array([bias, scale], dtype=np.int32)
    info = np.iinfo(out_dtype)
    lo, hi = (int(info.min), int(info.max)) if clamp is None else clamp
    p = Program()
    ia = p.binding(0, a.shape)
    inputs = [a]
    if constant_rhs:
        ib = b
    else:
        ib = p.binding(1, b.shape)
        inputs.append(b)
    oshape = ((B,) if (batch1 or batch2) else ()) + (M, N)
    out = p.binding(len(inputs), oshape, out_dtype)
    attrs = dict(output_zp=output_zp, output_min=lo, output_max=hi, shift=shift)
    p.matmul(ia, ib, sb, init=out, out_dtype=out_dtype, **attrs)
    attrs.update(input2=b, scale_bias=sb, out_dtype=out_dtype)
    return Workload("matmul_%dx%dx%dx%d" % (B, M, K, N), p, inputs, [(oshape, np.dtype(out_dtype).type)], 2 * B * M * K * N,
                    a.nbytes + b.nbytes + int(np.prod(oshape)) * np.dtype(out_dtype).itemsize, attrs)


def to_bf16(values):
    """float32 array -> bfloat16 bit patterns (uint16), round to nearest even."""
    f = np.ascontiguousarray(values, dtype=np.float32)
    u = f.reshape(-1).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = (u & 0x7fffffff) > 0x7f800000
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r.reshape(f.shape)


NO_CLAMP = (-8388608, 0x7f800000)  # float bit patterns of -inf / +inf, as the int32 attributes carry them


def float_bits(value):
    """The int32 attribute that carries a float clamp bound."""
    return int(np.array([value], dtype=np.float32).view(np.int32)[0])


def fully_connected_bf16_workload(M, K, N, seed=1010, clamp=None):
    """bf16 fully_connected (a linear layer of a decoder at M tokens): fp32 accumulate, float bias, bf16 out."""
    rng = np.random.default_rng(seed)
    x = to_bf16(rng.standard_normal((M, K)))
    w = to_bf16(rng.standard_normal((N, K)) / np.sqrt(K))
    bias = rng.standard_normal(N).astype(np.float32)
    lo, hi = NO_CLAMP if clamp is None else (float_bits(clamp[0]), float_bits(clamp[1]))
    attrs = dict(output_min=lo, output_max=hi)
    p = Program()
    inp = p.binding(0, (M, K), np.uint16)
    out = p.binding(1, (M, N), np.uint16)
    p.fully_connected(inp, w, bias, init=out, output_zp=0, shift_factor=0, input_zp=0, **attrs)
    bytes_ = x.nbytes + w.nbytes + bias.nbytes + 2 * M * N
    attrs.update(weights=w, bias=bias)
    return Workload("fcbf16_%dx%dx%d" % (M, K, N), p, [x], [((M, N), np.uint16)], 2 * M * K * N, bytes_, attrs)


def matmul_bf16_workload(B, M, K, N, batch1=True, batch2=True, constant_rhs=False, seed=1011, bias=0.0):
    """bf16 matmul [B,]M,K x [B,]K,N with one float bias; input2 a run-time binding unless constant_rhs."""
    rng = np.random.default_rng(seed)
    a = to_bf16(rng.standard_normal((B, M, K) if batch1 else (M, K)))
    b = to_bf16(rng.standard_normal((B, K, N) if batch2 else (K, N)) / np.sqrt(K))
    bv = np.array([bias], dtype=np.float32)
    p = Program()
    ia = p.binding(0, a.shape, np.uint16)
    inputs = [a]
    if constant_rhs:
        ib = b
    else:
        ib = p.binding(1, b.shape, np.uint16)
        inputs.append(b)
    oshape = ((B,) if (batch1 or batch2) else ()) + (M, N)
    out = p.binding(len(inputs), oshape, np.uint16)
    p.matmul(ia, ib, bv, init=out, output_zp=0, output_min=NO_CLAMP[0], output_max=NO_CLAMP[1], shift=0)
    attrs = dict(input2=b, bias=bv)
    return Workload("matmulbf16_%dx%dx%dx%d" % (B, M, K, N), p, inputs, [(oshape, np.uint16)], 2 * B * M * K * N,
                    a.nbytes + b.nbytes + 2 * int(np.prod(oshape)), attrs)


def conv2d_bf16_workload(N=1, H=14, W=14, C=16, O=24, KH=3, KW=3, stride=(1, 1), pad=(1, 1, 1, 1), nhwc=True, clamp=None,
                         depthwise=False, seed=1013):
    """bf16 conv2d (or depthwise_conv2d, O = C): fp32 accumulate, float bias, zero padding."""
    rng = np.random.default_rng(seed)
    x = to_bf16(rng.standard_normal((N, H, W, C)))
    if depthwise:
        O = C
        wts = to_bf16(rng.standard_normal((C, 1, KH, KW)) / np.sqrt(KH * KW))
    else:
        wts = to_bf16(rng.standard_normal((O, C, KH, KW)) / np.sqrt(C * KH * KW))
    bias = rng.standard_normal(O).astype(np.float32)
    lo, hi = NO_CLAMP if clamp is None else (float_bits(clamp[0]), float_bits(clamp[1]))
    if not nhwc:
        x = np.ascontiguousarray(x.transpose(0, 3, 1, 2))
    OH = (H + pad[2] + pad[3] - KH) // stride[0] + 1
    OW = (W + pad[0] + pad[1] - KW) // stride[1] + 1
    oshape = (N, OH, OW, O) if nhwc else (N, O, OH, OW)
    p = Program()
    inp = p.binding(0, x.shape, np.uint16)
    out = p.binding(1, oshape, np.uint16)
    fn = p.depthwise_conv2d if depthwise else p.conv2d
    fn(inp, wts, bias, init=out, input_zp=0, output_zp=0, output_min=lo, output_max=hi, shift_factor=0, pad=tuple(pad),
       stride=tuple(stride), nhwc_input=nhwc)
    macs = N * OH * OW * O * KH * KW * (1 if depthwise else C)
    attrs = dict(weights=wts, bias=bias, output_min=lo, output_max=hi, pad=tuple(pad), stride=tuple(stride), nhwc=nhwc)
    name = "%sbf16_%dx%dx%dx%d_o%d_k%dx%d_s%d" % ("dw" if depthwise else "conv", N, H, W, C, O, KH, KW, stride[0])
    return Workload(name, p, [x], [(oshape, np.uint16)], 2 * macs, x.nbytes + wts.nbytes + bias.nbytes + 2 * int(np.prod(oshape)), attrs)


def avg_pool2d_bf16_workload(N=2, H=7, W=7, C=1280, weight=None, clamp=None, seed=1014):
    """bf16 global average pool: one bf16 weight (1 / (H W) by default, the folded divide), bias 0."""
    rng = np.random.default_rng(seed)
    x = to_bf16(rng.standard_normal((N, H, W, C)) + 0.25)
    wt = to_bf16(np.array([1.0 / (H * W) if weight is None else weight]))
    bias = np.zeros(1, dtype=np.float32)
    lo, hi = NO_CLAMP if clamp is None else (float_bits(clamp[0]), float_bits(clamp[1]))
    p = Program()
    inp = p.binding(0, x.shape, np.uint16)
    out = p.binding(1, (N, 1, 1, C), np.uint16)
    p.avg_pool2d(inp, wt, bias, init=out, input_zp=0, output_zp=0, output_min=lo, output_max=hi, shift_factor=0)
    attrs = dict(weights=wt, bias=bias, output_min=lo, output_max=hi)
    return Workload("avgpoolbf16_%dx%dx%dx%d" % (N, H, W, C), p, [x], [((N, 1, 1, C), np.uint16)], 2 * x.size,
                    x.nbytes + 2 * N * C, attrs)


def expand_weights_workload(M=4, K=256, N=96, block=32, fold=True, clamp=None, expand_clamp=None, bias_pad=0, seed=1015):
    """Block-quantized int8 weights -> torq_hl.expand_weights -> bf16 matmul (fold=True: the expansion feeds only the
    matmul; False: it is also an output of the program, so it must run as an op of its own)."""
    rng = np.random.default_rng(seed)
    G = K // block
    x = to_bf16(rng.standard_normal((M, K)))
    wq = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
    scale = to_bf16(rng.uniform(0.5, 1.5, size=(G, N)) / (64.0 * np.sqrt(K)))
    zp = rng.integers(-8, 9, size=(G, N))
    cols = N + bias_pad
    qbias = np.zeros((G, cols), dtype=np.float32)
    qbias[:, :N] = (-zp).astype(np.float32) * from_bf16_np(scale)
    mm_bias = np.zeros(1, dtype=np.float32)
    lo, hi = NO_CLAMP if clamp is None else (float_bits(clamp[0]), float_bits(clamp[1]))
    elo, ehi = NO_CLAMP if expand_clamp is None else (float_bits(expand_clamp[0]), float_bits(expand_clamp[1]))
    p = Program()
    inp = p.binding(0, x.shape, np.uint16)
    out = p.binding(1, (M, N), np.uint16)
    outputs = [((M, N), np.uint16)]
    if fold:
        w16 = p.expand_weights(wq, scale, qbias, block_size=block, output_min=elo, output_max=ehi)
    else:
        wout = p.binding(2, (1, K, N), np.uint16)
        w16 = p.expand_weights(wq, scale, qbias, block_size=block, output_min=elo, output_max=ehi, init=wout)
        outputs.append(((1, K, N), np.uint16))
    p.matmul(inp, w16, mm_bias, init=out, output_zp=0, output_min=lo, output_max=hi, shift=0)
    attrs = dict(weights=wq, scale=scale, qbias=qbias, block=block, bias=mm_bias, output_min=lo, output_max=hi,
                 expand_min=elo, expand_max=ehi, fold=fold)
    return Workload("expandmm_%dx%dx%d_b%d%s" % (M, K, N, block, "" if fold else "_out"), p, [x], outputs, 2 * M * K * N,
                    x.nbytes + wq.nbytes + scale.nbytes + qbias.nbytes + 2 * M * N, attrs)


def from_bf16_np(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def add_bf16_workload(shape=(1, 32, 1152), w0=1.0, w1=1.0, bias=0.0, clamp=None, seed=1012):
    """bf16 add (a residual connection of a decoder layer): in1 * w0 + in2 * w1 + bias in fp32."""
    rng = np.random.default_rng(seed)
    a = to_bf16(rng.standard_normal(shape))
    b = to_bf16(rng.standard_normal(shape))
    wts = to_bf16(np.array([w0, w1], dtype=np.float32))
    bv = np.array([bias], dtype=np.float32)
    lo, hi = NO_CLAMP if clamp is None else (float_bits(clamp[0]), float_bits(clamp[1]))
    p = Program()
    out = p.binding(2, shape, np.uint16)
    p.add(p.binding(0, shape, np.uint16), p.binding(1, shape, np.uint16), wts, bv, init=out, output_zp=0, output_min=lo,
          output_max=hi, shift_factor=0)
    n = int(np.prod(shape))
    return Workload("addbf16_" + "x".join(str(d) for d in shape), p, [a, b], [(shape, np.uint16)], 3 * n, 6 * n,
                    dict(weights=wts, bias=bv, output_min=lo, output_max=hi))


def depthwise_workload(N=1, H=56, W=56, C=144, KH=3, KW=3, stride=(2, 2), pad=(0, 1, 0, 1), input_zp=-3,
                       output_zp=5, output_min=-128, output_max=127, realistic=True, nhwc=True, seed=1002, shift=None):
    """benchmark configuration 2a: depthwise 3x3 stride 2 SAME on 56x56x144.

    `shift` forces one shift_factor for every channel (multipliers drawn so that outputs still spread)."""
    rng = np.random.default_rng(seed)
    x = rng.integers(-128, 127, size=(N, H, W, C), endpoint=True, dtype=np.int8)
    w = rng.integers(-127, 127, size=(C, 1, KH, KW), endpoint=True, dtype=np.int8)
    tosa_bias = rng.integers(-(1 << 15), 1 << 15, size=C, endpoint=True, dtype=np.int64)
    if shift is not None:
        top = min(max(int(shift) - 10, 1), 31)
        mult = rng.integers(1 << (top - 1), (1 << top) - 1, size=C, endpoint=True, dtype=np.int64).astype(np.int32)
        shift = np.full(C, int(shift), dtype=np.int8)
    else:
        mult, shift = random_requant(rng, C, realistic)
        if realistic:
            shift = (shift - 4).astype(np.int8)  # only 9 taps: keep outputs spread over the int8 range
    sb, sf = derive_scale_bias(mult, shift, tosa_bias, w, input_zp)
    attrs = dict(input_zp=input_zp, output_zp=output_zp, output_min=output_min, output_max=output_max,
                 shift_factor=sf, pad=tuple(pad), stride=tuple(stride))
    p = Program()
    if not nhwc:
        x = np.ascontiguousarray(x.transpose(0, 3, 1, 2))
    inp = p.binding(0, x.shape)
    OH = (H + pad[2] + pad[3] - KH) // stride[0] + 1
    OW = (W + pad[0] + pad[1] - KW) // stride[1] + 1
    oshape = (N, OH, OW, C) if nhwc else (N, C, OH, OW)
    out = p.binding(1, oshape)
    p.depthwise_conv2d(inp, w, sb, init=out, nhwc_input=nhwc, **attrs)
    macs = N * OH * OW * C * KH * KW
    bytes_ = x.nbytes + w.nbytes + sb.nbytes + N * OH * OW * C
    attrs.update(weights=w, scale_bias=sb, nhwc=nhwc)
    return Workload("depthwise_%dx%dx%dx%d_k%dx%d_s%d" % (N, H, W, C, KH, KW, stride[0]), p, [x],
                    [(oshape, np.int8)], 2 * macs, bytes_, attrs)


def maxpool_workload(N=1, H=112, W=112, C=64, kernel=(2, 2), stride=(2, 2), pad=(0, 0, 0, 0), input_zp=-128,
                     nhwc=True, seed=1003):
    """benchmark configuration 2b: maxpool 2x2 stride 2 on 112x112x64."""
    rng = np.random.default_rng(seed)
    x = rng.integers(-128, 127, size=(N, H, W, C), endpoint=True, dtype=np.int8)
    attrs = dict(input_zp=input_zp, output_min=-128, output_max=127, stride=tuple(stride), pad=tuple(pad),
                 kernel=tuple(kernel))
    p = Program()
    if not nhwc:
        x = np.ascontiguousarray(x.transpose(0, 3, 1, 2))
    inp = p.binding(0, x.shape)
    OH = (H + pad[2] + pad[3] - kernel[0]) // stride[0] + 1
    OW = (W + pad[0] + pad[1] - kernel[1]) // stride[1] + 1
    oshape = (N, OH, OW, C) if nhwc else (N, C, OH, OW)
    out = p.binding(1, oshape)
    p.maxpool2d(inp, init=out, nhwc_input=nhwc, **attrs)
    attrs.update(nhwc=nhwc)
    return Workload("maxpool_%dx%dx%dx%d" % (N, H, W, C), p, [x], [(oshape, np.int8)],
                    N * OH * OW * C * kernel[0] * kernel[1], x.nbytes + N * OH * OW * C, attrs)


def copy_workload(nbytes=32 << 20, seed=1023):
    """A plain device copy through this library: a 1x1 stride-1 max pool over the whole int8 range (what a streaming
    kernel with no arithmetic reaches on this memory system; `nbytes` read and `nbytes` written)."""
    rng = np.random.default_rng(seed)
    pixels = nbytes // 64
    shape = (1, pixels // 1024, 1024, 64)
    x = rng.integers(-128, 127, size=shape, endpoint=True, dtype=np.int8)
    p = Program()
    inp = p.binding(0, shape)
    out = p.binding(1, shape)
    attrs = dict(input_zp=-128, output_min=-128, output_max=127, stride=(1, 1), pad=(0, 0, 0, 0), kernel=(1, 1))
    p.maxpool2d(inp, init=out, nhwc_input=True, **attrs)
    attrs.update(nhwc=True)
    return Workload("maxpool_copy_%dMiB" % (nbytes >> 20), p, [x], [(shape, np.int8)], x.size, 2 * x.nbytes, attrs)


def avgpool_workload(N=1, H=7, W=7, C=1280, input_zp=-3, output_zp=5, seed=1004):
    """benchmark configuration 2c: global average pool on 7x7x1280 (NHWC), scale = floor(2^20 / 49)."""
    rng = np.random.default_rng(seed)
    x = rng.integers(-128, 127, size=(N, H, W, C), endpoint=True, dtype=np.int8)
    # compiler/torq/Conversions/LinalgToTorqHL/PoolingPattern.cpp:325-328
    sb = np.array([-(H * W * input_zp), int((1 << 20) / (H * W))], dtype=np.int32)
    attrs = dict(input_zp=input_zp, output_zp=output_zp, output_min=-128, output_max=127, shift_factor=20)
    p = Program()
    inp = p.binding(0, x.shape)
    out = p.binding(1, (N, 1, 1, C))
    p.avg_pool2d(inp, np.array([1], dtype=np.int8), sb, init=out, **attrs)
    attrs.update(scale_bias=sb)
    return Workload("avgpool_%dx%dx%dx%d" % (N, H, W, C), p, [x], [((N, 1, 1, C), np.int8)], N * H * W * C,
                    x.nbytes + N * C, attrs)


def add_params(m0, m1, zp0, zp1, sign=1):
    """Quantised add parameters: compiler/torq/Conversions/LinalgToTorqHL/ElementWiseBinaryPattern.cpp:459-487."""
    S = 1 << 12
    w0 = np.int16(int(m0 * S))
    w1 = np.int16(int(m1 * S) * sign)
    bias = -int(m0 * S * zp0) - int(m1 * S * zp1) * sign
    return np.array([w0, w1], dtype=np.int16), np.array([bias, 1], dtype=np.int32), 12


def add_workload(N=1, H=56, W=56, C=24, zp0=-3, zp1=7, m0=0.71838506, m1=1.3 * 0.5, output_zp=-2, seed=1005):
    """benchmark configuration 2d: quantised add of two 56x56x24 tensors with distinct zero points and scales."""
    rng = np.random.default_rng(seed)
    a = rng.integers(-128, 127, size=(N, H, W, C), endpoint=True, dtype=np.int8)
    b = rng.integers(-128, 127, size=(N, H, W, C), endpoint=True, dtype=np.int8)
    wts, sb, sf = add_params(m0, m1, zp0, zp1)
    attrs = dict(output_zp=output_zp, output_min=-128, output_max=127, shift_factor=sf)
    p = Program()
    i0 = p.binding(0, a.shape)
    i1 = p.binding(1, b.shape)
    out = p.binding(2, a.shape)
    p.add(i0, i1, wts, sb, init=out, **attrs)
    attrs.update(weights=wts, scale_bias=sb)
    return Workload("add_%dx%dx%dx%d" % (N, H, W, C), p, [a, b], [(a.shape, np.int8)], 3 * a.size, 3 * a.nbytes,
                    attrs)


def branches_workload(M=64, K=256, N=128, seed=1030):
    """Three fully_connected records that read the same input and do not depend on each other, joined by two adds:
    out = add(add(fc_a(x), fc_b(x)), fc_c(x)).  A program with independent records (the shape of q / k / v projections
    or of a block with a projection shortcut)."""
    rng = np.random.default_rng(seed)
    x = rng.integers(-128, 127, size=(M, K), endpoint=True, dtype=np.int8)
    fcs = []
    for _ in range(3):
        wt = rng.integers(-128, 127, size=(N, K), endpoint=True, dtype=np.int8)
        mult, shift = random_requant(rng, N, True)
        sb, sf = derive_scale_bias(mult, shift, rng.integers(-(1 << 15), 1 << 15, size=N, endpoint=True, dtype=np.int64), wt, 0)
        fcs.append((wt, sb, dict(output_zp=int(rng.integers(-10, 10)), output_min=-128, output_max=127, shift_factor=sf)))
    adds = []
    for zp0, zp1 in ((fcs[0][2]["output_zp"], fcs[1][2]["output_zp"]), (-2, fcs[2][2]["output_zp"])):
        aw, asb, asf = add_params(0.71838506, 0.65, zp0, zp1)
        adds.append((aw, asb, dict(output_zp=-2, output_min=-128, output_max=127, shift_factor=asf)))
    p = Program()
    inp = p.binding(0, x.shape)
    out = p.binding(1, (M, N))
    ya, yb, yc = [p.fully_connected(inp, wt, sb, **at) for wt, sb, at in fcs]
    t = p.add(ya, yb, adds[0][0], adds[0][1], **adds[0][2])
    p.add(t, yc, adds[1][0], adds[1][1], init=out, **adds[1][2])
    return Workload("branches_%dx%dx%d" % (M, K, N), p, [x], [((M, N), np.int8)], 6 * M * K * N, x.nbytes + 3 * N * K + M * N,
                    dict(fcs=fcs, adds=adds))


def pointwise_add_workload(N=2, H=48, W=48, C=96, O=32, other_first=False, seed=1020):
    """The end of an inverted-residual block: 1x1 convolution -> add with a second input (the block's input)."""
    rng = np.random.default_rng(seed)
    x = rng.integers(-128, 127, size=(N, H, W, C), endpoint=True, dtype=np.int8)
    skip = rng.integers(-128, 127, size=(N, H, W, O), endpoint=True, dtype=np.int8)
    wp = rng.integers(-127, 127, size=(O, C, 1, 1), endpoint=True, dtype=np.int8)
    mult, shift = random_requant(rng, O, True)
    sbp, sfp = derive_scale_bias(mult, shift, rng.integers(-(1 << 15), 1 << 15, size=O, endpoint=True, dtype=np.int64), wp, 5)
    pattrs = dict(input_zp=5, output_zp=-7, output_min=-128, output_max=127, shift_factor=sfp, pad=(0, 0, 0, 0), stride=(1, 1))
    aw, asb, asf = add_params(0.71838506, 0.65, -3, -7) if other_first else add_params(0.65, 0.71838506, -7, -3)
    aattrs = dict(output_zp=-2, output_min=-128, output_max=127, shift_factor=asf)
    p = Program()
    inp = p.binding(0, x.shape)
    sk = p.binding(1, skip.shape)
    out = p.binding(2, skip.shape)
    t = p.conv2d(inp, wp, sbp, nhwc_input=True, **pattrs)
    if other_first:
        p.add(sk, t, aw, asb, init=out, **aattrs)
    else:
        p.add(t, sk, aw, asb, init=out, **aattrs)
    attrs = dict(pw=(wp, sbp, pattrs), add=(aw, asb, aattrs), other_first=other_first)
    return Workload("pwadd_%dx%dx%dx%d_o%d_%d" % (N, H, W, C, O, int(other_first)), p, [x, skip], [(skip.shape, np.int8)],
                    2 * N * H * W * C * O, x.nbytes + 2 * skip.nbytes + wp.nbytes, attrs)


_INT_RANGE = {np.dtype(np.int8): (-128, 127), np.dtype(np.int16): (-32768, 32767), np.dtype(np.int32): (-2 ** 31, 2 ** 31 - 1)}


def _random_ints(rng, shape, dtype, limit=None):
    lo, hi = _INT_RANGE[np.dtype(dtype)]
    if limit is not None:
        lo, hi = max(lo, -limit), min(hi, limit)
    return rng.integers(lo, hi, size=shape, endpoint=True, dtype=np.int64).astype(dtype)


def fma_workload(shape=(1, 56, 56, 24), in_dtype=np.int8, out_dtype=np.int8, input_zp=-3, scale=0.37, output_zp=5, weight=1, seed=1016):
    """Stand-alone rescale (tosa.rescale -> torq_hl.fma): weight 1, bias = -input_zp, TFLite multiplier / shift."""
    rng = np.random.default_rng(seed)
    x = _random_ints(rng, shape, in_dtype, limit=1 << 20)
    mult, sh = quantize_multiplier(scale)
    sb = np.array([-input_zp, int(mult)], dtype=np.int32)
    lo, hi = _INT_RANGE[np.dtype(out_dtype)]
    attrs = dict(output_zp=output_zp, output_min=lo, output_max=hi, shift_factor=int(sh))
    wts = np.array([weight], dtype=np.int8)
    p = Program()
    inp = p.binding(0, x.shape, in_dtype)
    out = p.binding(1, x.shape, out_dtype)
    p.fma(inp, wts, sb, init=out, **attrs)
    attrs.update(weights=wts, scale_bias=sb, out_dtype=out_dtype)
    nbytes = x.nbytes + x.size * np.dtype(out_dtype).itemsize
    return Workload("fma_%s_%s_%d" % (np.dtype(in_dtype).name, np.dtype(out_dtype).name, x.size), p, [x], [(x.shape, out_dtype)], 2 * x.size, nbytes, attrs)


def mul_workload(shape=(1, 56, 56, 24), in_dtype=np.int8, out_dtype=np.int8, scale=0.011, output_zp=-4, bias=0, broadcast=0, seed=1017):
    """Quantised multiply: inputs already zero-point free; one multiplier / shift.  broadcast 1 / 2: that input has one element."""
    rng = np.random.default_rng(seed)
    a = _random_ints(rng, (1,) if broadcast == 1 else shape, in_dtype)
    b = _random_ints(rng, (1,) if broadcast == 2 else shape, in_dtype)
    mult, sh = quantize_multiplier(scale)
    sb = np.array([bias, int(mult)], dtype=np.int32)
    lo, hi = _INT_RANGE[np.dtype(out_dtype)]
    attrs = dict(output_zp=output_zp, output_min=lo, output_max=hi, shift=int(sh))
    p = Program()
    i0 = p.binding(0, a.shape, in_dtype)
    i1 = p.binding(1, b.shape, in_dtype)
    out = p.binding(2, shape, out_dtype)
    p.mul(i0, i1, sb, init=out, **attrs)
    attrs.update(scale_bias=sb, out_dtype=out_dtype)
    count = int(np.prod(shape))
    nbytes = a.nbytes + b.nbytes + count * np.dtype(out_dtype).itemsize
    return Workload("mul_%s_%s_%d_b%d" % (np.dtype(in_dtype).name, np.dtype(out_dtype).name, count, broadcast), p, [a, b], [(shape, out_dtype)], 3 * count, nbytes, attrs)


def binary_workload(op_type=4, shape=(1, 56, 56, 24), dtype=np.int8, is_unsigned=False, seed=1021):
    """torq_hl.elementwisebinary: op_type 0 and, 1 or, 2 xor, 4 minimum, 5 maximum."""
    rng = np.random.default_rng(seed)
    a = _random_ints(rng, shape, dtype)
    b = _random_ints(rng, shape, dtype)
    p = Program()
    i0 = p.binding(0, shape, dtype)
    i1 = p.binding(1, shape, dtype)
    out = p.binding(2, shape, dtype)
    p.elementwisebinary(op_type, i0, i1, is_unsigned=is_unsigned, init=out)
    attrs = dict(op_type={0: "and", 1: "or", 2: "xor", 4: "minimum", 5: "maximum"}[op_type], is_unsigned=is_unsigned)
    return Workload("binary_%s_%s_%d_u%d" % (attrs["op_type"], np.dtype(dtype).name, a.size, int(is_unsigned)), p, [a, b], [(shape, dtype)], a.size,
                    3 * a.nbytes, attrs)


def compare_workload(op_type=6, shape=(1, 56, 56, 24), dtype=np.int8, is_unsigned=False, seed=1024):
    """torq_hl.elementwisebinary, comparison and logical modes: 6 greater, 7 greater-equal, 8 equal (integers in), 9 and,
    10 or, 11 xor (i1 in: uint8 0 / 1); the result is i1."""
    rng = np.random.default_rng(seed)
    if op_type >= 9:
        dtype = np.uint8
        a = rng.integers(0, 2, size=shape, dtype=np.uint8)
        b = rng.integers(0, 2, size=shape, dtype=np.uint8)
    else:
        a = _random_ints(rng, shape, dtype, limit=5)  # a narrow range: equal pairs do occur
        b = _random_ints(rng, shape, dtype, limit=5)
        _plant(a, [np.iinfo(dtype).min, np.iinfo(dtype).max, -1, 0])
        _plant(b, [np.iinfo(dtype).max, np.iinfo(dtype).min, 0, -1])
    p = Program()
    i0 = p.binding(0, shape, dtype)
    i1 = p.binding(1, shape, dtype)
    out = p.binding(2, shape, np.uint8)
    p.elementwisebinary(op_type, i0, i1, is_unsigned=is_unsigned, init=out)
    attrs = dict(op_type=op_type, is_unsigned=is_unsigned)
    return Workload("compare_%d_%s_%d_u%d" % (op_type, np.dtype(dtype).name, a.size, int(is_unsigned)), p, [a, b], [(shape, np.uint8)], a.size,
                    2 * a.nbytes + a.size, attrs)


def unary_workload(op_type=3, shape=(1, 56, 56, 24), dtype=np.int8, seed=1025):
    """torq_hl.elementwiseunary: 3 bitwise not (integers), 12 logical not (i1: uint8 0 / 1)."""
    rng = np.random.default_rng(seed)
    if op_type == 12:
        dtype = np.uint8
        a = rng.integers(0, 2, size=shape, dtype=np.uint8)
    else:
        a = _random_ints(rng, shape, dtype)
    p = Program()
    out = p.binding(1, shape, dtype)
    p.elementwiseunary(op_type, p.binding(0, shape, dtype), init=out)
    return Workload("unary_%d_%s_%d" % (op_type, np.dtype(dtype).name, a.size), p, [a], [(shape, np.dtype(dtype).type)], a.size, 2 * a.nbytes,
                    dict(op_type=op_type))


def shift_workload(op_type=2, shape=(1, 56, 56, 24), dtype=np.int32, round=True, seed=1026):
    """torq_hl.elementwiseshift: 0 logical right, 1 logical left, 2 arithmetic right; counts 0 .. bits-1 per element."""
    rng = np.random.default_rng(seed)
    a = _random_ints(rng, shape, dtype)
    bits = 8 * np.dtype(dtype).itemsize
    s = rng.integers(0, bits, size=shape).astype(dtype)
    _plant(a, [np.iinfo(dtype).min, np.iinfo(dtype).max, -1, 1, -3, 3])
    _plant(s, [bits - 1, bits - 1, 1, 1, 1, 1])
    p = Program()
    out = p.binding(2, shape, dtype)
    p.elementwiseshift(op_type, p.binding(0, shape, dtype), p.binding(1, shape, dtype), round=round, init=out)
    return Workload("shift_%d_%s_%d_r%d" % (op_type, np.dtype(dtype).name, a.size, int(round)), p, [a, s], [(shape, np.dtype(dtype).type)], a.size,
                    3 * a.nbytes, dict(op_type=op_type, round=round))


def _plant(a, values):
    """Writes the edge values into the first elements of `a` (as many as it has)."""
    flat = a.reshape(-1)
    n = min(flat.size, len(values))
    flat[:n] = values[:n]


def pack_table_words(lut):
    """Segment words of a 256-entry lookup table as the extract patterns build them
    (compiler/torq/Conversions/LinalgToTorqHL/ExtractPattern.cpp:30-54): sext(v) << 8 for int8, zext(v) for int16."""
    lut = np.asarray(lut)
    if lut.dtype == np.int8:
        return (lut.astype(np.int32) << 8).astype(np.int32)
    assert lut.dtype == np.int16
    return lut.view(np.uint16).astype(np.int32)


def table_workload(shape=(1, 56, 56, 24), in_dtype=np.int8, out_dtype=np.int8, static=False, seed=1027):
    """torq_hl.table: a random 256-entry lookup table of the output's type, as a constant operand or as the attribute."""
    rng = np.random.default_rng(seed)
    x = _random_ints(rng, shape, in_dtype)
    _plant(x, [-128, 127, 0, -1])
    lut = _random_ints(rng, (256,), out_dtype)
    lut[[0, 255]] = _INT_RANGE[np.dtype(out_dtype)]
    words = pack_table_words(lut)
    p = Program()
    out = p.binding(1, shape, out_dtype)
    p.table(p.binding(0, shape, in_dtype), [-128, 128], init=out, **({"static_table": words} if static else {"dynamic_table": words}))
    nbytes = x.nbytes + x.size * np.dtype(out_dtype).itemsize
    return Workload("table_%s_%s_%d_%s" % (np.dtype(in_dtype).name, np.dtype(out_dtype).name, x.size, "attr" if static else "operand"), p, [x],
                    [(shape, np.dtype(out_dtype).type)], x.size, nbytes, dict(words=words, lut=lut, out_dtype=out_dtype))


def act_workload(name="clamp", shape=(1, 56, 56, 24), in_dtype=np.int8, out_dtype=None, min_int=-20, max_int=90, seed=1018):
    """torq_hl.act on integers: clamp / abs / negate / i2i."""
    rng = np.random.default_rng(seed)
    out_dtype = in_dtype if out_dtype is None else out_dtype
    x = _random_ints(rng, shape, in_dtype)
    _plant(x, list(_INT_RANGE[np.dtype(in_dtype)]))  # the extremes: abs / negate of the most negative value saturate
    p = Program()
    inp = p.binding(0, x.shape, in_dtype)
    out = p.binding(1, x.shape, out_dtype)
    p.act(inp, name, min_int=min_int, max_int=max_int, init=out)
    attrs = dict(name=name, min_int=min_int, max_int=max_int, out_dtype=out_dtype)
    nbytes = x.nbytes + x.size * np.dtype(out_dtype).itemsize
    return Workload("act_%s_%s_%s_%d" % (name, np.dtype(in_dtype).name, np.dtype(out_dtype).name, x.size), p, [x], [(x.shape, out_dtype)], x.size, nbytes, attrs)


# ---------------------------------------------------------------------------------------------
# MobileNetV2-1.0 int8 (benchmark configuration 3)
# ---------------------------------------------------------------------------------------------
MBV2_BLOCKS = [(1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1)]


def quantize_multiplier(scale):
    """TFLite-style (multiplier in [2^30, 2^31], shift) with multiplier / 2^shift == scale."""
    m, e = np.frexp(np.asarray(scale, dtype=np.float64))
    mult = np.round(m * (1 << 31)).astype(np.int64)
    shift = 31 - e
    bump = mult == (1 << 31)
    mult = np.where(bump, mult // 2, mult)
    shift = np.where(bump, shift - 1, shift)
    return mult.astype(np.int32), shift.astype(np.int8)


def _same_pad(size, k, s):
    """TensorFlow SAME padding: (before, after)."""
    out = -(-size // s)
    total = max((out - 1) * s + k - size, 0)
    return total // 2, total - total // 2


class Layer:
    """One TorqHL op of a network workload: enough for the builder and for a checker to replay it."""

    def __init__(self, op, inputs, attrs, weights=None, scale_bias=None):
        self.op = op              # "conv2d" | "depthwise_conv2d" | "add" | "avg_pool2d" | "fully_connected" | "transpose"
        self.inputs = inputs      # indices into the tensor list (0 = network input)
        self.attrs = attrs
        self.weights = weights
        self.scale_bias = scale_bias


def mobilenet_v2_layers(resolution=224, classes=1000, seed=1006, width=1.0):
    """The layer list of MobileNetV2 with random int8 weights, int32 biases and per-channel requant
    parameters.  Scales are calibrated the way post-training quantisation does it: a float forward
    pass of one random image gives each layer's accumulator spread, and the per-channel scale maps
    it onto the int8 range, so no layer saturates or collapses."""
    import torch

    rng = np.random.default_rng(seed)
    layers = []
    shapes = [(resolution, resolution, 3)]  # H, W, C per tensor index
    zps = [int(rng.integers(-10, 10))]
    # calibration activations, N,C,H,W float64, already minus their zero point
    calib = [torch.from_numpy(rng.integers(-128, 127, size=(1, 3, resolution, resolution), endpoint=True).astype(np.float64) - zps[0])]

    def conv(src, O, k, s, relu6, depthwise=False):
        H, W, C = shapes[src]
        zp_in = zps[src]
        if depthwise:
            w = rng.integers(-127, 127, size=(C, 1, k, k), endpoint=True, dtype=np.int8)
            O_ = C
        else:
            w = rng.integers(-127, 127, size=(O, C, k, k), endpoint=True, dtype=np.int8)
            O_ = O
        pt, pb = _same_pad(H, k, s)
        pl, pr = _same_pad(W, k, s)
        tosa_bias = rng.integers(-(1 << 12), 1 << 12, size=O_, endpoint=True, dtype=np.int64)
        xp = torch.nn.functional.pad(calib[src], (pl, pr, pt, pb))  # x - zp is 0 in the padding
        acc = torch.nn.functional.conv2d(xp, torch.from_numpy(w.astype(np.float64)), stride=s, groups=C if depthwise else 1)
        acc = acc + torch.from_numpy(tosa_bias.astype(np.float64)).reshape(1, -1, 1, 1)
        spread = acc.std(dim=(0, 2, 3), unbiased=False).numpy() + 1.0  # a 1x1 frame has a spread of 0, not NaN
        # ReLU6 layers keep the positive half: give it most of the range; linear layers are centred
        eff = (60.0 if relu6 else 40.0) / spread * rng.uniform(0.8, 1.25, size=O_)
        mult, shift = quantize_multiplier(eff)
        sb, sf = derive_scale_bias(mult, shift, tosa_bias, w, zp_in)
        zp_out = int(rng.integers(-128, -110)) if relu6 else int(rng.integers(-20, 20))
        lo, hi = (zp_out if relu6 else -128), 127
        q = torch.clamp(torch.round(acc * torch.from_numpy(eff).reshape(1, -1, 1, 1)) + zp_out, lo, hi)
        OH, OW = -(-H // s), -(-W // s)
        attrs = dict(input_zp=zp_in, output_zp=zp_out, output_min=lo, output_max=hi,
                     shift_factor=sf, pad=(pl, pr, pt, pb), stride=(s, s))
        layers.append(Layer("depthwise_conv2d" if depthwise else "conv2d", [src], attrs, w, sb))
        shapes.append((OH, OW, O_))
        zps.append(zp_out)
        calib.append(q - zp_out)
        return len(shapes) - 1

    def add(a, b):
        zp_out = int(rng.integers(-20, 20))
        m0, m1 = float(rng.uniform(0.5, 0.8)), float(rng.uniform(0.5, 0.8))
        wts, sb, sf = add_params(m0, m1, zps[a], zps[b])
        layers.append(Layer("add", [a, b], dict(output_zp=zp_out, output_min=-128, output_max=127, shift_factor=sf), wts, sb))
        shapes.append(shapes[a])
        zps.append(zp_out)
        calib.append(torch.clamp(torch.round(calib[a] * m0 + calib[b] * m1) + zp_out, -128, 127) - zp_out)
        return len(shapes) - 1

    def ch(c):
        return max(8, int(c * width + 4) // 8 * 8)

    t = conv(0, ch(32), 3, 2, True)
    cin = ch(32)
    for expand, c, n, s in MBV2_BLOCKS:
        for i in range(n):
            stride = s if i == 0 else 1
            src = t
            h = conv(t, cin * expand, 1, 1, True) if expand != 1 else t
            h = conv(h, None, 3, stride, True, depthwise=True)
            h = conv(h, ch(c), 1, 1, False)
            t = add(src, h) if (stride == 1 and cin == ch(c)) else h
            cin = ch(c)
    t = conv(t, 1280, 1, 1, True)
    H, W, C = shapes[t]
    zp_out = int(rng.integers(-128, -110))
    sb = np.array([-(H * W * zps[t]), int((1 << 20) / (H * W))], dtype=np.int32)
    layers.append(Layer("avg_pool2d", [t], dict(input_zp=zps[t], output_zp=zp_out, output_min=-128, output_max=127,
                                                shift_factor=20), np.array([1], dtype=np.int8), sb))
    shapes.append((1, 1, C))
    zps.append(zp_out)
    pooled = calib[t].mean(dim=(2, 3))  # 1, C
    t = len(shapes) - 1
    w = rng.integers(-127, 127, size=(classes, C), endpoint=True, dtype=np.int8)
    tosa_bias = rng.integers(-(1 << 12), 1 << 12, size=classes, endpoint=True, dtype=np.int64)
    logits = pooled @ torch.from_numpy(w.astype(np.float64)).T
    eff = 40.0 / (float(logits.std()) + 1.0) * rng.uniform(0.8, 1.25, size=classes)
    mult, shift = quantize_multiplier(eff)
    sb, sf = derive_scale_bias(mult, shift, tosa_bias, w, zps[t])
    layers.append(Layer("fully_connected", [t], dict(output_zp=int(rng.integers(-20, 20)), output_min=-128, output_max=127,
                                                     shift_factor=sf), w, sb))
    shapes.append((1, 1, classes))
    return layers, shapes, zps[0]


def mobilenet_v2_workload(batch=1, resolution=224, classes=1000, seed=1006, nhwc=True, width=1.0):
    """benchmark configuration 3 as ONE program: 52 convs, 17 depthwise, 10 adds, global average pool, FC.

    nhwc=True declares every tensor N,H,W,C (the layout the kernels run); nhwc=False declares the ops
    N,C,H,W as the reference's patterns emit them, with the torq_hl.transpose the reference places in
    front of avg_pool2d."""
    layers, shapes, _ = mobilenet_v2_layers(resolution, classes, seed, width)
    rng = np.random.default_rng(seed + 1)
    H, W, C = shapes[0]
    x = rng.integers(-128, 127, size=(batch, H, W, C), endpoint=True, dtype=np.int8)
    if not nhwc:
        x = np.ascontiguousarray(x.transpose(0, 3, 1, 2))
    p = Program()
    vals = [p.binding(0, x.shape)]
    out_binding = p.binding(1, (batch, classes))
    macs = 0
    for li, L in enumerate(layers):
        src = [vals[i] for i in L.inputs]
        last = li == len(layers) - 1
        if L.op == "conv2d":
            v = p.conv2d(src[0], L.weights, L.scale_bias, nhwc_input=nhwc, **L.attrs)
            oh, ow, oc = shapes[li + 1]
            macs += batch * oh * ow * oc * int(np.prod(L.weights.shape[1:]))
        elif L.op == "depthwise_conv2d":
            v = p.depthwise_conv2d(src[0], L.weights, L.scale_bias, nhwc_input=nhwc, **L.attrs)
            oh, ow, oc = shapes[li + 1]
            macs += batch * oh * ow * oc * int(np.prod(L.weights.shape[2:]))
        elif L.op == "add":
            v = p.add(src[0], src[1], L.weights, L.scale_bias, **L.attrs)
        elif L.op == "avg_pool2d":
            s0 = src[0] if nhwc else p.transpose(src[0], (0, 2, 3, 1))
            v = p.avg_pool2d(s0, L.weights, L.scale_bias, **L.attrs)
        elif L.op == "fully_connected":
            v = p.fully_connected(src[0], L.weights, L.scale_bias, init=out_binding if last else None, **L.attrs)
            macs += batch * int(np.prod(L.weights.shape))
        else:
            raise ValueError(L.op)
        vals.append(v)
    wbytes = sum(L.weights.nbytes + L.scale_bias.nbytes for L in layers)
    wl = Workload("mobilenet_v2_b%d_%d" % (batch, resolution), p, [x], [((batch, classes), np.int8)], 2 * macs,
                  wbytes + x.nbytes + batch * classes, dict(layers=layers, shapes=shapes, nhwc=nhwc))
    return wl


# ---------------------------------------------------------------------------------------------------------------
# benchmark configuration 4: one decode step of a Gemma-3-1B-shaped decoder, the part of it that is on this path
# ---------------------------------------------------------------------------------------------------------------

class DecoderOp:
    """One TorqHL op of a decoder-step workload, by the names of the tensors it reads and writes, so that a checker
    can replay it (kind "linear": torq_hl.expand_weights folded into a bf16 torq_hl.matmul; "scores" / "context":
    the batched bf16 matmuls of the attention against the two caches; "add": bf16 torq_hl.add)."""

    def __init__(self, kind, out, inputs, shape, **params):
        self.kind = kind
        self.out = out
        self.inputs = inputs
        self.shape = tuple(shape)
        self.params = params


def _block_quantized(rng, K, N, block, gain):
    """int8 weights K x N, uniform in [-128, 127] (standard deviation 73.9), symmetric (no zero point, as the
    benchmark configuration says) with one bf16 scale per `block` input rows and output channel, drawn so that the
    expanded weights have a standard deviation of about gain / sqrt(K)."""
    wq = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
    scale = to_bf16(rng.uniform(0.75, 1.25, size=(K // block, N)) * (gain / (73.9 * np.sqrt(K))))
    return wq, scale, np.zeros((K // block, N), dtype=np.float32)


def decoder_step_workload(batch=1, layers=26, hidden=1152, heads=4, head_dim=256, ffn=6912, vocab=262144, cache_len=1024,
                          block=128, expose=False, seed=1040):
    """benchmark configuration 4 as ONE program: a decode step (one new token per sequence, `batch` sequences) of a
    decoder with `layers` layers, `heads` query heads over ONE key / value head, a gated feed-forward block and
    the vocabulary projection, on key / value caches of `cache_len` positions.

    Per layer, in data-flow order: q, k, v = x W (three bf16 matmuls whose int8 weights pass through
    torq_hl.expand_weights: bf16 scales per `block` input rows; k and v also leave the program, the caller appends
    them to its caches); scores = q K^T per sequence (torq_hl.matmul against the key cache, which is kept position-
    major [batch, cache_len, head_dim] and transposed by a torq_hl.transpose that the serialiser folds into the
    matmul); context = scores V (torq_hl.matmul against the value cache, kept dimension-major [batch, head_dim,
    cache_len] and transposed the same way); o = context W_o; h = add(x, o); gate, up = h W; a = add(gate, up);
    d = a W_down; x' = add(h, d).  Then logits = x W_vocab.  What a real decoder has between these ops -- the
    normalisations, the rotary embedding, the softmax over the scores, the gated activation and the embedding
    lookup -- are not ops of this path: scores feed the context matmul directly, the gate is an add, and the
    token embeddings arrive as the input binding.  Scales are chosen so that every tensor stays of order one.

    Bindings: 0 x [batch, hidden]; 1 key cache [layers * batch, cache_len, head_dim]; 2 value cache
    [layers * batch, head_dim, cache_len]; 3 logits [batch, vocab]; 4 new keys [layers, batch, head_dim];
    5 new values likewise; expose=True adds 6: every intermediate of every layer, one after another (wl.attrs
    ["trace"] maps names to (offset, shape)), so that each op can be checked on the inputs the GPU gave it."""
    rng = np.random.default_rng(seed)
    M, B = batch, batch
    qdim = heads * head_dim
    p = Program()
    p.set_name("decoder_step_b%d_l%d" % (batch, layers))
    x_in = to_bf16(rng.standard_normal((M, hidden)))
    kcache = to_bf16(rng.standard_normal((layers * B, cache_len, head_dim)))
    vcache = to_bf16(rng.standard_normal((layers * B, head_dim, cache_len)))
    bx = p.binding(0, x_in.shape, np.uint16)
    bk = p.binding(1, kcache.shape, np.uint16)
    bv = p.binding(2, vcache.shape, np.uint16)
    blog = p.binding(3, (M, vocab), np.uint16)
    bkn = p.binding(4, (layers, M, head_dim), np.uint16)
    bvn = p.binding(5, (layers, M, head_dim), np.uint16)
    trace, trace_elems = {}, 0
    per_layer = [("q", (M, qdim)), ("scores", (B, heads, cache_len)), ("context", (B, heads, head_dim)), ("o", (M, hidden)),
                 ("h", (M, hidden)), ("gate", (M, ffn)), ("up", (M, ffn)), ("a", (M, ffn)), ("d", (M, hidden)), ("x", (M, hidden))]
    if expose:
        for l in range(layers):
            for name, shape in per_layer:
                trace["%s%d" % (name, l)] = (trace_elems, shape)
                trace_elems += int(np.prod(shape))
        btrace = p.binding(6, (trace_elems,), np.uint16)
    zero = np.zeros(1, dtype=np.float32)
    noclamp = dict(output_zp=0, output_min=NO_CLAMP[0], output_max=NO_CLAMP[1])
    half = to_bf16(np.array([0.70703125, 0.70703125], dtype=np.float32))  # keeps a sum of two unit tensors at unit size
    ops, weight_bytes, macs = [], 0, 0

    def dest(name, shape):
        if not expose:
            return p.tensor(shape, np.uint16)
        off, _ = trace[name]
        return p.view(btrace, shape, off)

    def linear(out, src_name, src, K, N, gain, init=None):
        nonlocal weight_bytes, macs
        wq, scale, qbias = _block_quantized(rng, K, N, block, gain)
        w16 = p.expand_weights(wq, scale, qbias, block_size=block, output_min=NO_CLAMP[0], output_max=NO_CLAMP[1])
        y = p.matmul(src, w16, zero, init=init if init is not None else dest(out, (M, N)), shift=0, **noclamp)
        ops.append(DecoderOp("linear", out, [src_name], (M, N), weights=wq, scale=scale, qbias=qbias, block=block))
        weight_bytes += wq.nbytes
        macs += M * K * N
        return y

    def add(out, a_name, a, b_name, b, shape):
        y = p.add(a, b, half, zero, init=dest(out, shape), shift_factor=0, **noclamp)
        ops.append(DecoderOp("add", out, [a_name, b_name], shape, weights=half, bias=zero))
        return y

    x, xn = bx, "x_in"
    for l in range(layers):
        n = lambda s: "%s%d" % (s, l)
        q = linear(n("q"), xn, x, hidden, qdim, 1.0 / 512)
        linear(n("k"), xn, x, hidden, head_dim, 1.0, init=p.view(bkn, (M, head_dim), l * M * head_dim))
        linear(n("v"), xn, x, hidden, head_dim, 1.0, init=p.view(bvn, (M, head_dim), l * M * head_dim))
        keys = p.transpose(p.view(bk, (B, cache_len, head_dim), l * B * cache_len * head_dim), (0, 2, 1))
        scores = p.matmul(p.view(q, (B, heads, head_dim)), keys, zero, init=dest(n("scores"), (B, heads, cache_len)), shift=0, **noclamp)
        ops.append(DecoderOp("scores", n("scores"), [n("q")], (B, heads, cache_len), layer=l))
        values = p.transpose(p.view(bv, (B, head_dim, cache_len), l * B * head_dim * cache_len), (0, 2, 1))
        context = p.matmul(scores, values, zero, init=dest(n("context"), (B, heads, head_dim)), shift=0, **noclamp)
        ops.append(DecoderOp("context", n("context"), [n("scores")], (B, heads, head_dim), layer=l))
        macs += 2 * B * heads * cache_len * head_dim
        o = linear(n("o"), n("context"), p.view(context, (M, qdim)), qdim, hidden, 1.0)
        h = add(n("h"), xn, x, n("o"), o, (M, hidden))
        gate = linear(n("gate"), n("h"), h, hidden, ffn, 1.0)
        up = linear(n("up"), n("h"), h, hidden, ffn, 1.0)
        a = add(n("a"), n("gate"), gate, n("up"), up, (M, ffn))
        d = linear(n("d"), n("a"), a, ffn, hidden, 1.0)
        x = add(n("x"), n("h"), h, n("d"), d, (M, hidden))
        xn = n("x")
    linear("logits", xn, x, hidden, vocab, 1.0, init=blog)
    inputs = [x_in, kcache, vcache]
    outputs = [((M, vocab), np.uint16), ((layers, M, head_dim), np.uint16), ((layers, M, head_dim), np.uint16)]
    if expose:
        outputs.append(((trace_elems,), np.uint16))
    # algorithmic bytes: every int8 weight once (the figure a weight-streaming decode step is priced against), the
    # block scales, both caches and the activations that enter and leave
    scale_bytes = weight_bytes // block * 2
    bytes_ = weight_bytes + scale_bytes + kcache.nbytes + vcache.nbytes + x_in.nbytes + 2 * M * vocab + 4 * layers * M * head_dim
    attrs = dict(ops=ops, trace=trace, batch=batch, layers=layers, heads=heads, head_dim=head_dim, cache_len=cache_len,
                 hidden=hidden, ffn=ffn, vocab=vocab, weight_bytes=weight_bytes, expose=expose)
    return Workload("decoder_step_b%d_l%d" % (batch, layers), p, inputs, outputs, 2 * macs, bytes_, attrs)


def attention_workload(B=2, H=4, D=256, T=1024, D2=256, bias=(0.0, 0.0), clamp1=None, clamp2=None, rank2=False, seed=1045):
    """One decode step of attention as the decoder workload chains it: scores = q K^T against a key cache held
    [B, T, D], context = scores V against a value cache held dimension-major [B, D2, T] (both through a
    torq_hl.transpose that is read in place), the scores an intermediate nobody else reads.  Bindings: 0 q [B, H, D],
    1 keys, 2 values, 3 context [B, H, D2].  rank2: B == 1 with rank-2 operands."""
    rng = np.random.default_rng(seed)
    lead = () if rank2 else (B,)
    assert not rank2 or B == 1
    q = to_bf16(rng.standard_normal(lead + (H, D)))
    keys = to_bf16(rng.standard_normal(lead + (T, D)) / np.sqrt(D))
    vals = to_bf16(rng.standard_normal(lead + (D2, T)) / np.sqrt(T))
    perm = (1, 0) if rank2 else (0, 2, 1)
    p = Program()
    bq = p.binding(0, q.shape, np.uint16)
    bk = p.binding(1, keys.shape, np.uint16)
    bv = p.binding(2, vals.shape, np.uint16)
    out = p.binding(3, lead + (H, D2), np.uint16)
    lo1, hi1 = NO_CLAMP if clamp1 is None else (float_bits(clamp1[0]), float_bits(clamp1[1]))
    lo2, hi2 = NO_CLAMP if clamp2 is None else (float_bits(clamp2[0]), float_bits(clamp2[1]))
    scores = p.matmul(bq, p.transpose(bk, perm), np.array([bias[0]], np.float32), init=p.tensor(lead + (H, T), np.uint16), output_zp=0,
                      output_min=lo1, output_max=hi1, shift=0)
    p.matmul(scores, p.transpose(bv, perm), np.array([bias[1]], np.float32), init=out, output_zp=0, output_min=lo2, output_max=hi2, shift=0)
    attrs = dict(bias=bias, clamp1=(lo1, hi1), clamp2=(lo2, hi2))
    return Workload("attention_%dx%dx%dx%dx%d" % (B, H, D, T, D2), p, [q, keys, vals], [(lead + (H, D2), np.uint16)],
                    2 * B * H * T * (D + D2), 2 * (q.size + keys.size + vals.size + B * H * D2), attrs)


def grouped_linear_workload(M=3, K=256, N=64, mode="single", block=128, zero_points=False, clamp=None, expand_clamp=None, seed=1050):
    """Small programs of the shapes a decoder layer is made of, every result an output binding: mode "single" one
    linear; "concat" three linears (N, N / 2, N / 2 columns) on the same rows; "pair" two linears whose results an
    add joins (both also stored); "pair_hidden" the same with the two results intermediates that only the add
    reads; "residual" / "residual_first" a linear and the add of its result with (behind / in front of) the input
    rows (K == N).  zero_points: asymmetric quantisation (block biases -zp * scale, as the matmul patterns produce
    them).  attrs: ops (DecoderOp list), names (output names in binding order)."""
    rng = np.random.default_rng(seed)
    p = Program()
    x_in = to_bf16(rng.standard_normal((M, K)))
    bx = p.binding(0, (M, K), np.uint16)
    zero = np.zeros(1, dtype=np.float32)
    lo, hi = NO_CLAMP if clamp is None else (float_bits(clamp[0]), float_bits(clamp[1]))
    elo, ehi = NO_CLAMP if expand_clamp is None else (float_bits(expand_clamp[0]), float_bits(expand_clamp[1]))
    ops, names, outputs = [], [], []

    def out_binding(name, shape):
        names.append(name)
        outputs.append((shape, np.uint16))
        return p.binding(len(names), shape, np.uint16)

    def linear(name, n, init):
        wq = rng.integers(-128, 128, size=(K, n), dtype=np.int8)
        scale = to_bf16(rng.uniform(0.75, 1.25, size=(K // block, n)) / (73.9 * np.sqrt(K)))
        qbias = np.zeros((K // block, n), dtype=np.float32)
        if zero_points:
            qbias = (-rng.integers(-8, 9, size=(K // block, n))).astype(np.float32) * from_bf16_np(scale)
        w16 = p.expand_weights(wq, scale, qbias, block_size=block, output_min=elo, output_max=ehi)
        y = p.matmul(bx, w16, zero, init=init, output_zp=0, output_min=lo, output_max=hi, shift=0)
        ops.append(DecoderOp("linear", name, ["x_in"], (M, n), weights=wq, scale=scale, qbias=qbias, block=block, output_min=lo, output_max=hi,
                             expand_min=elo, expand_max=ehi))
        return y

    def add(name, a_name, a, b_name, b, shape):
        wts = to_bf16(np.array([0.75, -0.5], dtype=np.float32))
        bias = np.array([0.125], dtype=np.float32)
        y = p.add(a, b, wts, bias, init=out_binding(name, shape), output_zp=0, output_min=NO_CLAMP[0], output_max=NO_CLAMP[1], shift_factor=0)
        ops.append(DecoderOp("add", name, [a_name, b_name], shape, weights=wts, bias=bias))
        return y

    if mode == "single":
        linear("y", N, out_binding("y", (M, N)))
    elif mode == "concat":
        for i, n in enumerate((N, N // 2, N // 2)):
            linear("y%d" % i, n, out_binding("y%d" % i, (M, n)))
    elif mode in ("pair", "pair_hidden"):
        hidden = mode == "pair_hidden"
        g = linear("g", N, p.tensor((M, N), np.uint16) if hidden else out_binding("g", (M, N)))
        u = linear("u", N, p.tensor((M, N), np.uint16) if hidden else out_binding("u", (M, N)))
        add("a", "g", g, "u", u, (M, N))
    elif mode in ("residual", "residual_first"):
        assert K == N
        y = linear("y", N, out_binding("y", (M, N)))
        if mode == "residual":
            add("z", "y", y, "x_in", bx, (M, N))
        else:
            add("z", "x_in", bx, "y", y, (M, N))
    else:
        raise ValueError(mode)
    attrs = dict(ops=ops, names=names)
    name = "grouped_%s_%dx%dx%d_b%d%s" % (mode, M, K, N, block, "_zp" if zero_points else "")
    return Workload(name, p, [x_in], outputs, 2 * M * K * N, 0, attrs)
