"""Pins the op functions of the oracle against independent computations.

conv / depthwise accumulators: torch.nn.functional.conv2d on float64 (exact at these magnitudes)
and the pad-with-zero-point identity; fully_connected / matmul: numpy int64 matmul; maxpool: numpy
window maximum; avgpool / add / FC: known answers from the reference's fixture constants
(tests/golden/kat.json).  Requantisation in these checks is done by an independent numpy
restatement with exact integer arithmetic.
"""
import json
import os

import numpy as np
import pytest
import torch

from oracle import oracle as orc

KAT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "kat.json")))


def requant_np(acc, bias, scale, sh, zp, lo, hi):
    t1 = (acc.astype(object) + bias.astype(object)) * scale.astype(object)
    if sh > 0:
        t1 = t1 + (1 << (sh - 1))
    t3 = np.array([int(v) >> sh for v in t1.reshape(-1)], dtype=object).reshape(t1.shape)
    return np.clip((t3 + zp).astype(np.int64), lo, hi)


def rand_params(rng, ch, lo_shift=30, hi_shift=38):
    mult = rng.integers(1 << 30, (1 << 31) - 1, size=ch).astype(np.int32)
    shift = rng.integers(lo_shift, hi_shift, size=ch).astype(np.int8)
    return mult, shift


CONV_CASES = [
    # N, C, H, W, O, KH, KW, stride, pad[l,r,t,b]
    (1, 3, 8, 8, 4, 3, 3, (1, 1), (1, 1, 1, 1)),
    (2, 8, 9, 7, 5, 3, 3, (2, 2), (0, 1, 0, 1)),
    (1, 4, 10, 12, 6, 5, 2, (1, 1), (0, 0, 0, 0)),
    (1, 16, 6, 6, 8, 1, 1, (2, 2), (0, 0, 0, 0)),
    (1, 2, 7, 9, 3, 2, 5, (3, 4), (2, 1, 0, 3)),
]


@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("layout", [orc.NCHW, orc.NHWC])
def test_conv2d_against_torch(case, layout):
    N, C, H, W, O, KH, KW, stride, pad = case
    rng = np.random.default_rng(hash(case) & 0xffff)
    x = rng.integers(-128, 128, size=(N, C, H, W)).astype(np.int8)
    w = rng.integers(-127, 128, size=(O, C, KH, KW)).astype(np.int8)
    zp = -3
    tosa_bias = rng.integers(-(1 << 15), 1 << 15, size=O).astype(np.int32)
    mult, shift = rand_params(rng, O)
    sb, sf = orc.derive_scale_bias(mult, shift, tosa_bias, orc.per_channel_sum(w), zp)
    # independent accumulator: pad with zp, float64 conv
    pl, pr, pt, pb = pad
    xp = np.full((N, C, H + pt + pb, W + pl + pr), zp, dtype=np.float64)
    xp[:, :, pt:pt + H, pl:pl + W] = x
    acc = torch.nn.functional.conv2d(torch.from_numpy(xp), torch.from_numpy(w.astype(np.float64)), stride=stride)
    acc = acc.numpy().astype(np.int64)
    want = requant_np(acc, sb[0::2].reshape(1, O, 1, 1), sb[1::2].reshape(1, O, 1, 1), sf, 5, -128, 127).astype(np.int8)
    xin = x if layout == orc.NCHW else np.ascontiguousarray(x.transpose(0, 2, 3, 1))
    got = orc.conv2d(xin, w, sb, input_zp=zp, output_zp=5, output_min=-128, output_max=127, shift_factor=sf,
                     pad=pad, stride=stride, layout=layout)
    if layout == orc.NHWC:
        got = got.transpose(0, 3, 1, 2)
    assert np.array_equal(got, want)


def test_conv2d_pad_with_zero_point_identity():
    """conv(pad_zp(x), w) + (b - zp*sum(w)) == conv(pad_0(x - zp), w) + b  (why bias carries -zp*sum w)."""
    rng = np.random.default_rng(3)
    x = rng.integers(-128, 128, size=(1, 5, 6, 6)).astype(np.int8)
    w = rng.integers(-127, 128, size=(4, 5, 3, 3)).astype(np.int8)
    zp = 7
    tosa_bias = rng.integers(-1000, 1000, size=4).astype(np.int32)
    one = np.full(4, 1, dtype=np.int32)
    sb = np.empty(8, dtype=np.int32)
    sb[0::2] = tosa_bias - zp * orc.per_channel_sum(w)
    sb[1::2] = one
    got = orc.conv2d(x, w, sb, input_zp=zp, output_zp=0, output_min=-(1 << 31), output_max=(1 << 31) - 1,
                     shift_factor=0, pad=(1, 1, 1, 1), stride=(1, 1), out_dtype=np.int32)
    xc = torch.from_numpy(x.astype(np.float64) - zp)
    want = torch.nn.functional.conv2d(xc, torch.from_numpy(w.astype(np.float64)), padding=1).numpy().astype(np.int64)
    want = want + tosa_bias.reshape(1, 4, 1, 1)
    assert np.array_equal(got.astype(np.int64), want)


@pytest.mark.parametrize("layout", [orc.NCHW, orc.NHWC])
@pytest.mark.parametrize("geom", [(3, 3, (1, 1), (1, 1, 1, 1)), (3, 3, (2, 2), (0, 1, 0, 1)), (4, 4, (2, 2), (1, 2, 1, 2)), (1, 5, (1, 1), (2, 2, 0, 0))])
def test_depthwise_against_torch(layout, geom):
    KH, KW, stride, pad = geom
    rng = np.random.default_rng(11)
    N, C, H, W = 2, 6, 9, 10
    x = rng.integers(-128, 128, size=(N, C, H, W)).astype(np.int8)
    w = rng.integers(-127, 128, size=(C, 1, KH, KW)).astype(np.int8)
    zp = 4
    mult, shift = rand_params(rng, C, 28, 34)
    sb, sf = orc.derive_scale_bias(mult, shift, rng.integers(-500, 500, size=C).astype(np.int32), orc.per_channel_sum(w), zp)
    pl, pr, pt, pb = pad
    xp = np.full((N, C, H + pt + pb, W + pl + pr), zp, dtype=np.float64)
    xp[:, :, pt:pt + H, pl:pl + W] = x
    acc = torch.nn.functional.conv2d(torch.from_numpy(xp), torch.from_numpy(w.astype(np.float64)), stride=stride, groups=C)
    acc = acc.numpy().astype(np.int64)
    want = requant_np(acc, sb[0::2].reshape(1, C, 1, 1), sb[1::2].reshape(1, C, 1, 1), sf, -1, -128, 127).astype(np.int8)
    xin = x if layout == orc.NCHW else np.ascontiguousarray(x.transpose(0, 2, 3, 1))
    got = orc.depthwise_conv2d(xin, w, sb, input_zp=zp, output_zp=-1, output_min=-128, output_max=127,
                               shift_factor=sf, pad=pad, stride=stride, layout=layout)
    if layout == orc.NHWC:
        got = got.transpose(0, 3, 1, 2)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("mkn", [(1, 1, 1), (3, 61, 19), (16, 128, 40), (5, 700, 33)])
def test_fully_connected_against_numpy(mkn):
    M, K, N = mkn
    rng = np.random.default_rng(M * 131 + K)
    x = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    w = rng.integers(-128, 128, size=(N, K)).astype(np.int8)
    mult, shift = rand_params(rng, N, 32, 40)
    sb, sf = orc.derive_scale_bias(mult, shift, rng.integers(-9999, 9999, size=N).astype(np.int32), None, 0)
    acc = x.astype(np.int64) @ w.astype(np.int64).T
    want = requant_np(acc, sb[0::2][None], sb[1::2][None], sf, 2, -128, 127).astype(np.int8)
    got = orc.fully_connected(x, w, sb, output_zp=2, output_min=-128, output_max=127, shift_factor=sf)
    assert np.array_equal(got, want)


def test_fully_connected_known_answers():
    k = KAT["fc_conv1d_matmul_fc_requant"]
    x = np.array(k["inputs"], dtype=np.int8)
    w = np.array(k["weights_fk"], dtype=np.int8)
    sb, sf = orc.derive_scale_bias(np.array(k["multiplier"], dtype=np.int32), np.array(k["shift"], dtype=np.int8),
                                   np.array(k["tosa_bias"], dtype=np.int32), None, 0)
    assert sb.tolist() == k["scale_bias"] and sf == k["shift_factor"]
    got = orc.fully_connected(x, w, sb, output_zp=k["output_zp"], output_min=k["output_min"],
                              output_max=k["output_max"], shift_factor=sf)
    assert got.tolist() == k["expected"]


@pytest.mark.parametrize("bshape", [((4, 5), (5, 3)), ((2, 4, 5), (2, 5, 3)), ((1, 4, 8), (3, 8, 2)), ((3, 4, 8), (8, 2))])
def test_matmul_against_numpy(bshape):
    sa, sbb = bshape
    rng = np.random.default_rng(5)
    a = rng.integers(-128, 128, size=sa).astype(np.int8)
    b = rng.integers(-128, 128, size=sbb).astype(np.int8)
    acc = np.matmul(a.astype(np.int64), b.astype(np.int64))
    acc = acc.reshape((-1,) + acc.shape[-2:])
    got = orc.matmul(a, b, np.array([0, 1], dtype=np.int32), output_zp=0, output_min=-(1 << 31),
                     output_max=(1 << 31) - 1, shift=0, out_dtype=np.int32)
    assert np.array_equal(got.astype(np.int64), acc)
    # one (bias, scale) pair for every column
    got8 = orc.matmul(a, b, np.array([17, 3 << 20], dtype=np.int32), output_zp=-4, output_min=-128,
                      output_max=127, shift=30, out_dtype=np.int8)
    want8 = requant_np(acc, np.array(17), np.array(3 << 20), 30, -4, -128, 127).astype(np.int8)
    assert np.array_equal(got8, want8)


@pytest.mark.parametrize("geom", [((2, 2), (2, 2), (0, 0, 0, 0)), ((3, 3), (2, 2), (1, 1, 1, 1)), ((3, 3), (1, 1), (0, 0, 0, 0)), ((1, 3), (1, 3), (0, 2, 0, 0)), ((5, 5), (5, 5), (0, 0, 0, 0))])
@pytest.mark.parametrize("layout", [orc.NCHW, orc.NHWC])
def test_maxpool_against_numpy(geom, layout):
    kernel, stride, pad = geom
    rng = np.random.default_rng(9)
    N, C, H, W = 2, 5, 10, 11
    x = rng.integers(-128, 128, size=(N, C, H, W)).astype(np.int8)
    zp = -128
    pl, pr, pt, pb = pad
    xp = np.full((N, C, H + pt + pb, W + pl + pr), zp, dtype=np.int64)
    xp[:, :, pt:pt + H, pl:pl + W] = x
    OH = (H + pt + pb - kernel[0]) // stride[0] + 1
    OW = (W + pl + pr - kernel[1]) // stride[1] + 1
    want = np.empty((N, C, OH, OW), dtype=np.int8)
    for oy in range(OH):
        for ox in range(OW):
            win = xp[:, :, oy * stride[0]:oy * stride[0] + kernel[0], ox * stride[1]:ox * stride[1] + kernel[1]]
            want[:, :, oy, ox] = win.max(axis=(2, 3))
    xin = x if layout == orc.NCHW else np.ascontiguousarray(x.transpose(0, 2, 3, 1))
    got = orc.maxpool2d(xin, input_zp=zp, output_min=-128, output_max=127, stride=stride, pad=pad, kernel=kernel,
                        layout=layout)
    if layout == orc.NHWC:
        got = got.transpose(0, 3, 1, 2)
    assert np.array_equal(got, want)


def test_maxpool_padding_value_is_input_zp():
    x = np.full((1, 1, 2, 2), -100, dtype=np.int8)
    got = orc.maxpool2d(x, input_zp=-50, output_min=-128, output_max=127, stride=(2, 2), pad=(1, 1, 1, 1), kernel=(2, 2))
    assert got.tolist() == [[[[-50, -50], [-50, -50]]]]


def test_avgpool_known_answers():
    k = KAT["avgpool_7x7"]
    sb, sf = orc.derive_avgpool_params(k["H"], k["W"], k["input_zp"])
    assert sb.tolist() == k["scale_bias"] and sf == k["shift_factor"]
    for v, want in zip(k["constant_inputs"], k["expected"]):
        x = np.full((1, k["H"], k["W"], 3), v, dtype=np.int8)
        got = orc.avg_pool2d(x, sb, output_zp=k["output_zp"], output_min=k["output_min"], output_max=k["output_max"], shift_factor=sf)
        assert got.reshape(-1).tolist() == [want] * 3


def test_avgpool_close_to_true_mean_and_exact_to_formula():
    rng = np.random.default_rng(2)
    x = rng.integers(-128, 128, size=(3, 7, 7, 40)).astype(np.int8)
    zp_in, zp_out = -3, 5
    sb, sf = orc.derive_avgpool_params(7, 7, zp_in)
    got = orc.avg_pool2d(x, sb, output_zp=zp_out, output_min=-128, output_max=127, shift_factor=sf)
    acc = x.astype(np.int64).sum(axis=(1, 2))
    want = requant_np(acc, np.array(sb[0]), np.array(sb[1]), sf, zp_out, -128, 127).astype(np.int8)
    assert np.array_equal(got.reshape(3, 40), want)
    true = np.clip(np.floor((acc - 49 * zp_in) / 49 + 0.5) + zp_out, -128, 127)
    assert np.abs(got.reshape(3, 40).astype(np.int64) - true).max() <= 1


def test_add_known_answers():
    k = KAT["add_tosa_add_mlir"]
    w, sb, sf = orc.derive_add_params(k["m0"], k["m1"], k["zp0"], k["zp1"])
    assert w.tolist() == k["weights"] and sb.tolist() == k["scale_bias"] and sf == k["shift_factor"]
    a = np.array([p[0] for p in k["inputs"]], dtype=np.int8)
    b = np.array([p[1] for p in k["inputs"]], dtype=np.int8)
    got = orc.add(a, b, w, sb, output_zp=k["output_zp"], output_min=k["output_min"], output_max=k["output_max"], shift_factor=sf)
    assert got.tolist() == k["expected"]


def test_add_half_half_closed_form():
    # m0 = m1 = 1/2, zero points 0: q = round_half_up((a + b) / 2)
    w, sb, sf = orc.derive_add_params(0.5, 0.5, 0, 0)
    assert w.tolist() == [2048, 2048] and sb.tolist() == [0, 1] and sf == 12
    a = np.arange(-128, 128, dtype=np.int64)
    aa, bb = np.meshgrid(a, a)
    got = orc.add(aa.astype(np.int8), bb.astype(np.int8), w, sb, output_zp=0, output_min=-128, output_max=127, shift_factor=sf)
    want = np.clip(np.floor((aa + bb) / 2 + 0.5), -128, 127)
    assert np.array_equal(got.astype(np.int64), want.astype(np.int64))


def test_add_rejects_int16_overflow_and_sub_sign():
    assert orc.derive_add_params(9.0, 0.5, 0, 0) is None
    w, sb, _ = orc.derive_add_params(0.5, 0.25, 3, -5, sign=-1)
    assert w.tolist() == [2048, -1024]
    assert sb[0] == -int(0.5 * 4096 * 3) + int(0.25 * 4096 * -5)
