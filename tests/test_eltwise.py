"""Integer elementwise ops next to the convolution path: torq_hl.fma (the stand-alone rescale), torq_hl.mul and
torq_hl.act (clamp / abs / negate / i2i).  Oracle pins, the emitter, and (on a GPU) the kernel, bit-exact."""
import numpy as np
import pytest

import desc_interp
from helpers import assert_bit_exact, families, oracle_eval, run_on_gpu
from oracle import oracle as orc
from torq_compiler_amd import Program, ThipError, runtime, workloads as w


def _r1_exact(acc, bias, scale, shift, zp, lo, hi):
    """The ACT stage with Python integers: floor((t0 * scale) / 2^shift + 1/2) as an exact rational."""
    t1 = (int(acc) + int(bias)) * int(scale)
    t3 = (2 * t1 + (1 << shift)) // (1 << (shift + 1)) if shift > 0 else t1
    return min(max(t3 + zp, lo), hi)


# ---- oracle pins ----------------------------------------------------------------------------------------
def test_fma_is_the_exact_rescale():
    """Every int8 input (and a sweep of int16 / int32 ones) against exact integer arithmetic; scale = 2^shift with
    weight 1 is x - input_zp + output_zp."""
    x8 = np.arange(-128, 128, dtype=np.int8)
    for shift, scale, bias, zp, weight in [(31, 1 << 30, 3, -2, 1), (38, 1518500250, -7, 11, 1), (12, 2896, 0, 0, -3), (0, 5, 1, 0, 2), (45, 2 ** 31 - 1, 100, -128, 1)]:
        got = orc.fma(x8, [weight], [bias, scale], output_zp=zp, output_min=-128, output_max=127, shift_factor=shift)
        want = [_r1_exact(int(v) * weight, bias, scale, shift, zp, -128, 127) for v in x8]
        assert got.tolist() == want, (shift, scale)
    got = orc.fma(x8, [1], [5, 1 << 20], output_zp=-9, output_min=-2 ** 31, output_max=2 ** 31 - 1, shift_factor=20, out_dtype=np.int32)
    assert np.array_equal(got, x8.astype(np.int32) + 5 - 9)
    rng = np.random.default_rng(3)
    x32 = rng.integers(-2 ** 20, 2 ** 20, size=500).astype(np.int32)
    got = orc.fma(x32, [1], [-17, 1330000000], output_zp=3, output_min=-32768, output_max=32767, shift_factor=37, out_dtype=np.int16)
    assert got.tolist() == [_r1_exact(int(v), -17, 1330000000, 37, 3, -32768, 32767) for v in x32]
    x16 = rng.integers(-32768, 32768, size=500).astype(np.int16)
    got = orc.fma(x16, [1], [128, 1 << 30], output_zp=-128, output_min=-128, output_max=127, shift_factor=38)
    assert got.tolist() == [_r1_exact(int(v), 128, 1 << 30, 38, -128, -128, 127) for v in x16]


def test_mul_against_exact_products():
    """All 65 536 int8 pairs, random int16 pairs, and both broadcasts."""
    a, b = np.meshgrid(np.arange(-128, 128, dtype=np.int8), np.arange(-128, 128, dtype=np.int8))
    for shift, scale, bias, zp in [(37, 1503238554, 0, -4), (20, 1 << 13, 9, 0), (33, 2 ** 31 - 1, -300, 7)]:
        got = orc.mul(a, b, [bias, scale], output_zp=zp, output_min=-128, output_max=127, shift=shift)
        t1 = (a.astype(np.int64) * b.astype(np.int64) + bias) * scale
        want = np.clip(((t1 + (1 << (shift - 1))) >> shift) + zp, -128, 127)  # int64 cannot overflow at these sizes
        assert np.array_equal(got, want.astype(np.int8)), (shift, scale)
        sample = [(5, 77), (200, 13), (255, 255), (0, 0), (128, 64)]
        assert [int(got[i, j]) for i, j in sample] == [_r1_exact(int(a[i, j]) * int(b[i, j]), bias, scale, shift, zp, -128, 127) for i, j in sample]
    rng = np.random.default_rng(4)
    x, y = rng.integers(-32768, 32768, size=400).astype(np.int16), rng.integers(-32768, 32768, size=400).astype(np.int16)
    got = orc.mul(x, y, [0, 1 << 30], output_zp=0, output_min=-32768, output_max=32767, shift=45, out_dtype=np.int16)
    assert got.tolist() == [_r1_exact(int(p) * int(q), 0, 1 << 30, 45, 0, -32768, 32767) for p, q in zip(x, y)]
    one = np.array([-7], dtype=np.int16)
    assert np.array_equal(orc.mul(x, one, [0, 1], output_zp=0, output_min=-2 ** 31, output_max=2 ** 31 - 1, shift=0, out_dtype=np.int32), x.astype(np.int32) * -7)
    assert np.array_equal(orc.mul(one, x, [0, 1], output_zp=0, output_min=-2 ** 31, output_max=2 ** 31 - 1, shift=0, out_dtype=np.int32), x.astype(np.int32) * -7)


def test_act_modes():
    x = np.arange(-128, 128, dtype=np.int8)
    assert np.array_equal(orc.act(x, "clamp", min_int=-20, max_int=90), np.clip(x, -20, 90))
    assert np.array_equal(orc.act(x, "abs"), np.minimum(np.abs(x.astype(np.int32)), 127).astype(np.int8))      # |-128| saturates
    assert np.array_equal(orc.act(x, "negate"), np.minimum(-x.astype(np.int32), 127).astype(np.int8))
    assert np.array_equal(orc.act(x, "abs", out_dtype=np.int16), np.abs(x.astype(np.int16)))                    # the wider type holds 128
    wide = np.array([-2 ** 31, -70000, -129, -1, 0, 127, 128, 65535, 2 ** 31 - 1], dtype=np.int32)
    assert np.array_equal(orc.act(wide, "i2i", out_dtype=np.int8), wide.astype(np.int8))                        # truncation, no clipping
    assert np.array_equal(orc.act(wide, "i2i", out_dtype=np.int16), wide.astype(np.int16))
    assert np.array_equal(orc.act(x, "i2i", out_dtype=np.int32), x.astype(np.int32))
    assert np.array_equal(orc.act(wide, "negate"), np.clip(-wide.astype(np.int64), -2 ** 31, 2 ** 31 - 1).astype(np.int32))
    assert np.array_equal(orc.act(wide, "clamp", min_int=-100, max_int=100, out_dtype=np.int8), np.clip(wide, -100, 100).astype(np.int8))


def test_elementwise_binary_modes():
    rng = np.random.default_rng(6)
    for dt in (np.int8, np.int16, np.int32):
        info = np.iinfo(dt)
        a = rng.integers(info.min, info.max, size=300, endpoint=True).astype(dt)
        b = rng.integers(info.min, info.max, size=300, endpoint=True).astype(dt)
        a[:3], b[:3] = [info.min, info.max, -1], [info.max, info.min, 0]
        assert np.array_equal(orc.elementwise_binary("and", a, b), a & b)
        assert np.array_equal(orc.elementwise_binary("or", a, b), a | b)
        assert np.array_equal(orc.elementwise_binary("xor", a, b), a ^ b)
        assert np.array_equal(orc.elementwise_binary("minimum", a, b), np.minimum(a, b))
        assert np.array_equal(orc.elementwise_binary("maximum", a, b), np.maximum(a, b))
    a16, b16 = a.astype(np.int16), b.astype(np.int16)
    assert np.array_equal(orc.elementwise_binary("minimum", a16, b16, is_unsigned=True).view(np.uint16), np.minimum(a16.view(np.uint16), b16.view(np.uint16)))
    assert np.array_equal(orc.elementwise_binary("maximum", a16, b16, is_unsigned=True).view(np.uint16), np.maximum(a16.view(np.uint16), b16.view(np.uint16)))


# ---- emitter ----------------------------------------------------------------------------------------------
CASES = [lambda: w.fma_workload(), lambda: w.fma_workload((3, 5, 7), np.int16, np.int8, input_zp=11, scale=0.004, output_zp=-128),
         lambda: w.fma_workload((1000,), np.int32, np.int16, scale=0.0021, output_zp=0), lambda: w.fma_workload((37,), np.int8, np.int32, scale=3.7, weight=-2),
         lambda: w.fma_workload((4, 33), np.int8, np.int16, scale=2.0 ** -20),
         lambda: w.mul_workload(), lambda: w.mul_workload((2, 9, 13), np.int16, np.int8, scale=2.0 ** -22, output_zp=3),
         lambda: w.mul_workload((129,), np.int8, np.int32, scale=0.5, bias=-5), lambda: w.mul_workload((5, 17), np.int16, np.int16, scale=2.0 ** -15, broadcast=2),
         lambda: w.mul_workload((64,), np.int8, np.int8, scale=0.02, broadcast=1),
         lambda: w.act_workload("clamp"), lambda: w.act_workload("abs"), lambda: w.act_workload("negate", (77,), np.int16),
         lambda: w.act_workload("i2i", (5, 9), np.int32, np.int8), lambda: w.act_workload("i2i", (50,), np.int8, np.int32),
         lambda: w.act_workload("abs", (19,), np.int8, np.int16), lambda: w.act_workload("clamp", (300,), np.int32, np.int16, min_int=-32768, max_int=1000),
         lambda: w.binary_workload(0), lambda: w.binary_workload(1, (77,), np.int16), lambda: w.binary_workload(2, (5, 9), np.int32),
         lambda: w.binary_workload(4), lambda: w.binary_workload(5, (1000,), np.int16, is_unsigned=True), lambda: w.binary_workload(4, (333,), np.int16, is_unsigned=True),
         lambda: w.binary_workload(5, (4099,), np.int32)]


@pytest.mark.parametrize("make", CASES)
def test_eltwise_descriptor(make):
    wl = make()
    outs = [np.zeros(s, dtype=dt) for s, dt in wl.outputs]
    d = desc_interp.run(wl.program.serialize(), list(wl.inputs) + outs)
    assert_bit_exact(outs[0], oracle_eval(wl)[0], wl.name)
    assert [int(o["kind"]) for o in d.ops] == [desc_interp.K_ELTWISE]


def test_eltwise_in_a_program():
    """conv2d -> act(clamp) -> fma -> mul with the conv's own output: intermediates, not bindings."""
    conv = w.conv2d_workload(N=1, H=12, W=12, C=16, O=32, nhwc=True)
    rng = np.random.default_rng(8)
    x = conv.inputs[0]
    p = Program()
    inp = p.binding(0, x.shape)
    a = conv.attrs
    y = p.conv2d(inp, a["weights"], a["scale_bias"], input_zp=a["input_zp"], output_zp=a["output_zp"], output_min=a["output_min"], output_max=a["output_max"],
                 shift_factor=a["shift_factor"], pad=a["pad"], stride=a["stride"], nhwc_input=True)
    c = p.act(y, "clamp", min_int=-50, max_int=60)
    r = p.fma(c, np.array([1], dtype=np.int8), np.array([7, 1 << 30], dtype=np.int32), output_zp=-1, output_min=-128, output_max=127, shift_factor=31)
    out = p.binding(1, y.shape)
    p.mul(r, y, np.array([0, 1 << 24], dtype=np.int32), output_zp=2, output_min=-128, output_max=127, shift=30, init=out)
    got = np.zeros(y.shape, dtype=np.int8)
    d = desc_interp.run(p.serialize(), [x, got])
    y0 = oracle_eval(conv)[0]
    c0 = orc.act(y0, "clamp", min_int=-50, max_int=60)
    r0 = orc.fma(c0, [1], [7, 1 << 30], output_zp=-1, output_min=-128, output_max=127, shift_factor=31)
    want = orc.mul(r0, y0, [0, 1 << 24], output_zp=2, output_min=-128, output_max=127, shift=30)
    assert_bit_exact(got, want, "conv -> clamp -> fma -> mul")
    assert [int(o["kind"]) for o in d.ops][-3:] == [desc_interp.K_ELTWISE] * 3
    del rng


def test_eltwise_rejections():
    def expect(code, build):
        p = Program()
        with pytest.raises(ThipError) as e:
            build(p)
            p.serialize()
        assert e.value.code == code, e.value

    sb = np.array([0, 1], dtype=np.int32)
    one = np.array([1], dtype=np.int8)
    ok = dict(output_zp=0, output_min=-128, output_max=127)
    expect(runtime.INVALID_ARGUMENT, lambda p: p.fma(p.binding(0, (8,)), one, sb, init=p.binding(1, (9,)), shift_factor=1, **ok))
    expect(runtime.INVALID_ARGUMENT, lambda p: p.fma(p.binding(0, (8,)), one, sb, init=p.binding(1, (8,)), shift_factor=64, **ok))
    expect(runtime.INVALID_ARGUMENT, lambda p: p.fma(p.binding(0, (8,)), one, sb, init=p.binding(1, (8,)), shift_factor=1, output_zp=0, output_min=-129, output_max=127))
    expect(runtime.UNIMPLEMENTED, lambda p: p.fma(p.binding(0, (8,), np.uint16), one, sb, init=p.binding(1, (8,)), shift_factor=1, **ok))
    expect(runtime.UNIMPLEMENTED, lambda p: p.mul(p.binding(0, (8,)), p.binding(1, (8,), np.int16), sb, init=p.binding(2, (8,)), shift=1, **ok))
    expect(runtime.UNIMPLEMENTED, lambda p: p.mul(p.binding(0, (8,)), p.binding(1, (4,)), sb, init=p.binding(2, (8,)), shift=1, **ok))
    expect(runtime.UNIMPLEMENTED, lambda p: p.act(p.binding(0, (8,)), "ceil", init=p.binding(1, (8,))))
    expect(runtime.UNIMPLEMENTED, lambda p: p.act(p.binding(0, (8,)), "i2i", init=p.binding(1, (8,)), weights=one))
    expect(runtime.INVALID_ARGUMENT, lambda p: p.act(p.binding(0, (8,)), "clamp", min_int=-200, max_int=5, init=p.binding(1, (8,))))
    expect(runtime.INVALID_ARGUMENT, lambda p: p.act(p.binding(0, (8,)), "clamp", min_int=6, max_int=5, init=p.binding(1, (8,))))
    expect(runtime.UNIMPLEMENTED, lambda p: p.elementwisebinary(6, p.binding(0, (8,)), p.binding(1, (8,)), init=p.binding(2, (8,))))   # GREATER
    expect(runtime.UNIMPLEMENTED, lambda p: p.elementwisebinary(runtime.MINIMUM, p.binding(0, (8,)), p.binding(1, (8,)), is_unsigned=True, init=p.binding(2, (8,))))
    expect(runtime.UNIMPLEMENTED, lambda p: p.elementwisebinary(runtime.MAXIMUM, p.binding(0, (8,)), p.binding(1, (8,), np.int16), init=p.binding(2, (8,))))
    expect(runtime.INVALID_ARGUMENT, lambda p: p.elementwisebinary(runtime.MAXIMUM, p.binding(0, (8,)), p.binding(1, (9,)), init=p.binding(2, (8,))))


TRANSPOSES = [((5, 9), (1, 0), np.int8), ((70, 130), (1, 0), np.uint16), ((3, 33, 65), (0, 2, 1), np.int16), ((2, 5, 6, 7), (0, 2, 3, 1), np.int8),
              ((2, 6, 7, 5), (0, 3, 1, 2), np.uint16), ((1, 24, 56, 56), (0, 2, 3, 1), np.int8)]


def _transpose_program(shape, perm, dtype, seed=9):
    rng = np.random.default_rng(seed)
    info = np.iinfo(dtype)
    x = rng.integers(info.min, info.max, size=shape, endpoint=True).astype(dtype)
    p = Program()
    out_shape = tuple(shape[i] for i in perm)
    p.transpose(p.binding(0, shape, dtype), perm, init=p.binding(1, out_shape, dtype))
    return p, x, np.ascontiguousarray(x.transpose(perm))


@pytest.mark.parametrize("shape,perm,dtype", TRANSPOSES)
def test_transpose_op_descriptor(shape, perm, dtype):
    """torq_hl.transpose between bindings, 8- and 16-bit elements (bf16 bit patterns travel as uint16)."""
    p, x, want = _transpose_program(shape, perm, dtype)
    got = np.zeros(want.shape, dtype=dtype)
    d = desc_interp.run(p.serialize(), [x, got])
    assert np.array_equal(got, want)
    assert [int(o["kind"]) for o in d.ops] == [desc_interp.K_TRANSPOSE]


# ---- GPU ---------------------------------------------------------------------------------------------------
@pytest.mark.gpu
def test_gpu_transpose_op(device):
    from torq_compiler_amd import Executable
    for shape, perm, dtype in TRANSPOSES + [((4, 144, 28, 28), (0, 2, 3, 1), np.uint16), ((1000, 3000), (1, 0), np.int8)]:
        p, x, want = _transpose_program(shape, perm, dtype)
        print("[gpu-case] transpose", shape, perm, np.dtype(dtype).name, flush=True)
        exe = Executable(device, p.serialize())
        got = np.zeros(want.shape, dtype=dtype)
        exe.run_host([x, got])
        exe.close()
        assert np.array_equal(got, want)



@pytest.mark.gpu
def test_gpu_eltwise(device):
    """Every case of the emitter test, plus sizes that exercise whole vectors, the ragged tail and both requant tails
    (shift below and above 33)."""
    extra = [lambda: w.fma_workload((64, 56, 56, 24)), lambda: w.fma_workload((100003,), np.int16, np.int8, scale=0.0009, output_zp=-7),
             lambda: w.fma_workload((4099,), np.int8, np.int8, scale=2.0 ** -3), lambda: w.mul_workload((64, 56, 56, 24)),
             lambda: w.mul_workload((70001,), np.int16, np.int8, scale=2.0 ** -21, broadcast=2), lambda: w.mul_workload((1031,), np.int8, np.int16, scale=0.3),
             lambda: w.act_workload("abs", (64, 56, 56, 24)), lambda: w.act_workload("i2i", (9999,), np.int32, np.int8)]
    for make in CASES + extra:
        wl = make()
        print("[gpu-case]", wl.name, flush=True)
        got, kernels = run_on_gpu(device, wl, via="device" if wl.inputs[0].size > 5000 else "host")
        assert_bit_exact(got[0], oracle_eval(wl)[0], wl.name)
        assert families(kernels) == ["eltwise_int"]


@pytest.mark.gpu
def test_gpu_eltwise_kernel_does_not_depend_on_where_a_binding_lies(device):
    """Device bindings need 16-byte alignment and nothing more: the kernel an executable names when it is created is the
    one that runs for bindings at any such address (the vector width is bounded by those 16 bytes), results included."""
    from torq_compiler_amd import Executable
    for wl in (w.act_workload("i2i", (9999,), np.int32, np.int8), w.fma_workload((4099,), np.int16, np.int8, scale=0.0009, output_zp=-7),
               w.act_workload("abs", (777,), np.int32, np.int32)):
        exe = Executable(device, wl.program.serialize())
        named = exe.op_kernels()
        assert named[0].startswith("eltwise_int<") and not named[0].endswith(",1>"), named
        want = oracle_eval(wl)[0]
        for offset in (0, 16, 48):
            x = wl.inputs[0]
            src = device.alloc(x.nbytes + 64)
            dst = device.alloc(want.nbytes + 64)
            staged = device.upload(x)
            # upload() gives a fresh allocation; place the input at the offset through a second copy on the host side
            host = np.zeros(x.nbytes + 64, dtype=np.uint8)
            host[offset:offset + x.nbytes] = x.reshape(-1).view(np.uint8)
            device.free(staged)
            runtime.check(runtime.lib().thip_device_h2d(device.handle, src, host.ctypes.data, host.nbytes))
            exe.run_device([src + offset, dst + offset], [x.nbytes, want.nbytes])
            got = device.download(dst, (want.nbytes + 64,), np.uint8)[offset:offset + want.nbytes].view(want.dtype).reshape(want.shape)
            assert_bit_exact(got, want, "%s at +%d" % (wl.name, offset))
            assert exe.op_kernels() == named
            device.free(src)
            device.free(dst)
        exe.close()


# ---- comparisons, logical ops, bitwise not, shifts ------------------------------------------------------------------
def test_oracle_compare_logical_and_not():
    """What pins them is the arith op each mode replaces (ArithToTorqHLPattern.cpp:104-131,181-251): numpy's comparison /
    logical functions on every int8 pair, on int16 / int32 extremes, and on the unsigned views of 16-bit operands."""
    a8, b8 = np.meshgrid(np.arange(-128, 128, dtype=np.int8), np.arange(-128, 128, dtype=np.int8))
    for mode, fn in [(6, np.greater), (7, np.greater_equal), (8, np.equal)]:
        assert np.array_equal(orc.elementwise_compare(mode, a8, b8), fn(a8, b8).astype(np.uint8))
        for dt in (np.int16, np.int32):
            info = np.iinfo(dt)
            x = np.array([info.min, info.max, -1, 0, 1, info.min, 7, -7], dtype=dt)
            y = np.array([info.max, info.min, 0, -1, 1, info.min, -7, 7], dtype=dt)
            assert np.array_equal(orc.elementwise_compare(mode, x, y), fn(x, y).astype(np.uint8))
        x = np.array([-1, 0, 1, -32768, 32767, 5], dtype=np.int16)
        y = np.array([1, -1, 1, 32767, -32768, 5], dtype=np.int16)
        assert np.array_equal(orc.elementwise_compare(mode, x, y, is_unsigned=True), fn(x.view(np.uint16), y.view(np.uint16)).astype(np.uint8))
    t = np.array([0, 0, 1, 1], dtype=np.uint8)
    u = np.array([0, 1, 0, 1], dtype=np.uint8)
    assert orc.elementwise_compare(9, t, u).tolist() == [0, 0, 0, 1]
    assert orc.elementwise_compare(10, t, u).tolist() == [0, 1, 1, 1]
    assert orc.elementwise_compare(11, t, u).tolist() == [0, 1, 1, 0]
    assert orc.elementwise_unary(12, t).tolist() == [1, 1, 0, 0]
    for dt in (np.int8, np.int16, np.int32):
        info = np.iinfo(dt)
        x = np.array([info.min, info.max, -1, 0, 1, 85], dtype=dt)
        assert np.array_equal(orc.elementwise_unary(3, x), np.invert(x))
        assert np.array_equal(orc.elementwise_unary(3, orc.elementwise_unary(3, x)), x)


def test_oracle_shifts():
    """The rounding right shift is the linalg body the reference's pattern matches (ArithToTorqHLPattern.cpp:367-379):
    (x >> s) + (s > 0 and bit s-1 of x); checked against exact rationals floor(x / 2^s + 1/2) with Python integers, the
    logical forms on the unsigned bit patterns, the left shift modulo the width."""
    for dt, bits in ((np.int8, 8), (np.int16, 16), (np.int32, 32)):
        info = np.iinfo(dt)
        rng = np.random.default_rng(bits)
        xs = np.concatenate([np.array([info.min, info.max, -1, 0, 1, -3, 3, -2, 2, -5, 5], dtype=dt),
                             rng.integers(info.min, info.max, size=300, endpoint=True, dtype=np.int64).astype(dt)])
        for s in list(range(bits)):
            sv = np.full(xs.shape, s, dtype=dt)
            px = [int(v) for v in xs]
            ux = [v & ((1 << bits) - 1) for v in px]
            wrap = lambda v: ((v + (1 << (bits - 1))) % (1 << bits)) - (1 << (bits - 1))
            assert orc.elementwise_shift(2, xs, sv, round=False).tolist() == [v >> s for v in px]
            assert orc.elementwise_shift(2, xs, sv, round=True).tolist() == [wrap((2 * v + (1 << s)) >> (s + 1)) if s else v for v in px]
            assert orc.elementwise_shift(0, xs, sv, round=False).tolist() == [wrap(v >> s) for v in ux]
            assert orc.elementwise_shift(0, xs, sv, round=True).tolist() == [wrap((2 * v + (1 << s)) >> (s + 1)) if s else wrap(v) for v in ux]
            assert orc.elementwise_shift(1, xs, sv).tolist() == [wrap((v << s) & ((1 << bits) - 1)) for v in ux]
    # the matched body itself, on int32
    x = np.array([5, -5, 6, -6, 7, -7, 2 ** 31 - 1, -2 ** 31], dtype=np.int64)
    for s in (1, 2, 5, 31):
        body = (x >> s) + (((x >> (s - 1)) & 1) if s > 0 else 0)
        got = orc.elementwise_shift(2, x.astype(np.int32), np.full(8, s, dtype=np.int32), round=True)
        assert got.tolist() == [int(((v + 2 ** 31) % 2 ** 32) - 2 ** 31) for v in body]


NEW_ELTWISE = [lambda: w.compare_workload(6), lambda: w.compare_workload(7, dtype=np.int16), lambda: w.compare_workload(8, dtype=np.int32),
               lambda: w.compare_workload(6, dtype=np.int16, is_unsigned=True), lambda: w.compare_workload(7, shape=(3, 7, 11), dtype=np.int8),
               lambda: w.compare_workload(9), lambda: w.compare_workload(10, shape=(5, 13)), lambda: w.compare_workload(11),
               lambda: w.unary_workload(3), lambda: w.unary_workload(3, dtype=np.int16, shape=(3, 5, 7)), lambda: w.unary_workload(3, dtype=np.int32),
               lambda: w.unary_workload(12),
               lambda: w.shift_workload(2, round=True), lambda: w.shift_workload(2, dtype=np.int16, round=False), lambda: w.shift_workload(0, dtype=np.int8, round=True),
               lambda: w.shift_workload(0, dtype=np.int32, round=False), lambda: w.shift_workload(1, dtype=np.int16, shape=(7, 9)), lambda: w.shift_workload(1)]


@pytest.mark.parametrize("make", NEW_ELTWISE)
def test_new_eltwise_descriptors(make):
    wl = make()
    blob = wl.program.serialize()
    outs = [np.zeros(s, dtype=dt) for s, dt in wl.outputs]
    d = desc_interp.run(blob, list(wl.inputs) + outs)
    assert_bit_exact(outs[0], oracle_eval(wl)[0], wl.name)
    assert [int(o["kind"]) for o in d.ops] == [desc_interp.K_ELTWISE]


def test_new_eltwise_rejections():
    p = Program()
    a = p.binding(0, (4, 4), np.int8)
    with pytest.raises(ThipError):
        p.elementwiseshift(3, a, p.binding(1, (4, 4), np.int8), init=p.binding(2, (4, 4), np.int8))  # ASL is not lowered
        p.serialize()
    p = Program()
    a = p.binding(0, (4, 4), np.int8)
    with pytest.raises(ThipError):
        p.elementwisebinary(6, a, p.binding(1, (4, 4), np.int8), init=p.binding(2, (4, 4), np.int8))  # a comparison gives i1
        p.serialize()
    p = Program()
    with pytest.raises(ThipError):
        p.elementwiseunary(12, p.binding(0, (4, 4), np.int8), init=p.binding(1, (4, 4), np.int8))  # LOGICAL_NOT is for i1
        p.serialize()
    p = Program()
    with pytest.raises(ThipError):
        p.elementwisebinary(13, p.binding(0, (4,), np.int32), p.binding(1, (4,), np.int32), init=p.binding(2, (4,), np.int32))  # 48-bit SUB
        p.serialize()


@pytest.mark.gpu
@pytest.mark.parametrize("make", NEW_ELTWISE + [lambda: w.compare_workload(6, shape=(64, 56, 56, 24)), lambda: w.shift_workload(2, shape=(8, 56, 56, 24), round=True)])
def test_gpu_new_eltwise(device, make):
    wl = make()
    print("[gpu-case]", wl.name, flush=True)
    got, kernels = run_on_gpu(device, wl, via="device" if wl.inputs[0].size > 10000 else "host")
    assert_bit_exact(got[0], oracle_eval(wl)[0], wl.name)
    assert families(kernels) == ["eltwise_int"]


# ---- torq_hl.table: the plain lookups the extract patterns produce --------------------------------------------------

def test_oracle_table_is_the_lookup_of_the_program_it_replaces():
    """The reference rewrites `extract(lut, index_cast(x) + 128)` into torq_hl.table with the words of
    ExtractPattern.cpp:30-54 and scale_bias [-128, 128] (:56-62), so the op must give lut[x + 128]: checked for every
    int8 input against plain indexing, for int8 and int16 tables, and for int16 inputs through their low byte
    (the trunci of :485-497)."""
    rng = np.random.default_rng(7)
    x8 = np.arange(-128, 128, dtype=np.int8)
    for dtype in (np.int8, np.int16):
        info = np.iinfo(dtype)
        lut = rng.integers(info.min, info.max, size=256, endpoint=True).astype(dtype)
        lut[:2] = [info.min, info.max]
        words = w.pack_table_words(lut)
        # the packing itself, against the pattern's arithmetic written out
        want_words = [(int(v) << 8) & 0xFFFFFFFF if dtype == np.int8 else int(v) & 0xFFFF for v in lut]
        assert [int(t) & 0xFFFFFFFF for t in words] == want_words
        np.testing.assert_array_equal(orc.table(x8, words, dtype), lut[x8.astype(np.int64) + 128])
    x16 = rng.integers(-32768, 32767, size=4096, endpoint=True).astype(np.int16)
    np.testing.assert_array_equal(orc.table(x16, words, np.int16), lut[x16.astype(np.int8).astype(np.int64) + 128])
    # the slope half of a word never contributes while the fraction is zero
    noisy = (words.astype(np.int64) & 0xFFFF | (rng.integers(0, 1 << 16, size=256) << 16)).astype(np.uint32).view(np.int32)
    np.testing.assert_array_equal(orc.table(x8, noisy, np.int16), lut[x8.astype(np.int64) + 128])


def test_oracle_table_refuses_what_the_sources_do_not_define():
    words = w.pack_table_words(np.arange(-128, 128, dtype=np.int8))
    x = np.arange(-128, 128, dtype=np.int8)
    with pytest.raises(ValueError):
        orc.table(x, words, np.int8, bias=0, scale=1)  # a 9.7 input with a fraction: interpolation
    with pytest.raises(ValueError):
        orc.table(x, words + 1, np.int8)  # an int8 result from a base with a low byte
    with pytest.raises(ValueError):
        orc.table(x, words, np.int8, bias=128, scale=128)  # entries 256 .. 511 of a 256-entry table


TABLES = [lambda: w.table_workload(), lambda: w.table_workload(static=True), lambda: w.table_workload(out_dtype=np.int16, shape=(3, 7, 11)),
          lambda: w.table_workload(in_dtype=np.int16, out_dtype=np.int16, static=True), lambda: w.table_workload(shape=(1, 1, 1, 5))]


@pytest.mark.parametrize("make", TABLES)
def test_table_descriptor(make):
    wl = make()
    blob = wl.program.serialize()
    outs = [np.zeros(s, dtype=dt) for s, dt in wl.outputs]
    d = desc_interp.run(blob, list(wl.inputs) + outs)
    assert_bit_exact(outs[0], oracle_eval(wl)[0], wl.name)
    np.testing.assert_array_equal(outs[0], wl.attrs["lut"][(wl.inputs[0].astype(np.int64) & 0xFF) ^ 0x80])
    assert [(int(o["kind"]), int(o["variant"])) for o in d.ops] == [(desc_interp.K_ELTWISE, 22)]


def test_table_rejections():
    words = w.pack_table_words(np.arange(-128, 128, dtype=np.int8))

    def build(scale_bias=(-128, 128), in_dtype=np.int8, out_dtype=np.int8, **table):
        p = Program()
        p.table(p.binding(0, (4, 4), in_dtype), list(scale_bias), init=p.binding(1, (4, 4), out_dtype), **table)
        return p.serialize()

    build(dynamic_table=words)
    for bad in (dict(scale_bias=(0, 1), dynamic_table=words),          # an interpolated lookup
                dict(dynamic_table=words[:128]),                       # not 256 entries
                dict(dynamic_table=words + 3),                         # int8 result from a base with a low byte
                dict(in_dtype=np.int16, dynamic_table=words),          # int16 -> int8 is not a form the patterns produce
                dict(out_dtype=np.int32, dynamic_table=words),
                dict(dynamic_table=words, static_table=words),         # both forms at once
                dict()):                                               # no table
        with pytest.raises(ThipError):
            build(**bad)
    p = Program()
    with pytest.raises(ThipError):  # a run-time table is torq_hl.gather in the reference
        op = runtime.HlTable(p.binding(1, (4, 4), np.int8).index, p.constant(np.array([-128, 128], dtype=np.int32)).index,
                             p.binding(0, (4, 4), np.int8).index, p.binding(2, (256,), np.int32).index, None, 0)
        runtime.check(runtime.lib().thip_hl_table(p._h, __import__("ctypes").byref(op)))
        p.serialize()


@pytest.mark.gpu
@pytest.mark.parametrize("make", TABLES + [lambda: w.table_workload(shape=(64, 56, 56, 24)), lambda: w.table_workload(shape=(8, 56, 56, 24), out_dtype=np.int16)])
def test_gpu_table(device, make):
    wl = make()
    print("[gpu-case]", wl.name, flush=True)
    got, kernels = run_on_gpu(device, wl, via="device" if wl.inputs[0].size > 10000 else "host")
    assert_bit_exact(got[0], oracle_eval(wl)[0], wl.name)
    assert families(kernels) == ["table_lookup"]


# ---- tensors of one to five elements --------------------------------------------------------------------------------

TINY = [lambda sh=sh, f=f: f(sh) for sh in [(1,), (2,), (3,), (5,), (1, 1, 3)] for f in (
    lambda sh: w.shift_workload(0, shape=sh, dtype=np.int16, round=True, seed=1),
    lambda sh: w.binary_workload(4, shape=sh, dtype=np.int8, seed=2),
    lambda sh: w.compare_workload(7, shape=sh, dtype=np.int32, seed=3),
    lambda sh: w.table_workload(shape=sh, seed=4),
    lambda sh: w.act_workload("abs", shape=sh, in_dtype=np.int8, min_int=-5, max_int=90, seed=5),
    lambda sh: w.fma_workload(sh, in_dtype=np.int8, out_dtype=np.int16, input_zp=3, scale=0.7, output_zp=-4, seed=6))]


@pytest.mark.parametrize("make", TINY)
def test_tiny_tensors_descriptor(make):
    """The generators plant their edge values into as many elements as the tensor has; the record covers the ragged tail."""
    wl = make()
    outs = [np.zeros(s, dtype=dt) for s, dt in wl.outputs]
    desc_interp.run(wl.program.serialize(), list(wl.inputs) + outs)
    assert_bit_exact(outs[0], oracle_eval(wl)[0], wl.name)


@pytest.mark.gpu
def test_gpu_tiny_tensors(device):
    for make in TINY:
        wl = make()
        print("[gpu-case]", wl.name, wl.inputs[0].shape, flush=True)
        got, _ = run_on_gpu(device, wl, via="host")
        assert_bit_exact(got[0], oracle_eval(wl)[0], wl.name)
