"""Host logic: the emitter's packing, k-table, scale_bias split and layout folding, checked on the CPU.

The descriptor is executed by the numpy interpreter in desc_interp.py (test-only) and compared
bit-for-bit with the oracle.  Geometries follow the ones the reference's own tests exercise
(tests/models/keras_conv.py, keras_pointwise.py, keras_depthwise.py, keras_fc.py, keras_pooling.py,
tests/testdata/tosa_ops/*.mlir).
"""
import numpy as np
import pytest

import desc_interp
from helpers import assert_bit_exact, oracle_eval
from oracle import oracle as orc
from torq_compiler_amd import Program, ThipError, runtime, workloads as w


def interp(wl):
    blob = wl.program.serialize()
    outs = [np.zeros(s, dtype=dt) for s, dt in wl.outputs]
    d = desc_interp.run(blob, list(wl.inputs) + outs)
    return outs, d


CONV = [
    dict(N=1, H=8, W=8, C=3, O=4, KH=3, KW=3),
    dict(N=1, H=8, W=8, C=4, O=8, KH=2, KW=3, pad=(0, 0, 0, 0)),
    dict(N=1, H=12, W=12, C=1, O=4, KH=6, KW=6, stride=(2, 2), pad=(2, 2, 2, 2)),
    dict(N=1, H=18, W=76, C=24, O=7, KH=5, KW=2, pad=(0, 1, 2, 2)),
    dict(N=1, H=9, W=9, C=8, O=16, KH=1, KW=1, stride=(2, 2), pad=(0, 0, 0, 0)),
    dict(N=2, H=5, W=5, C=16, O=29, KH=3, KW=5, stride=(3, 4), pad=(2, 2, 1, 1)),
    dict(N=1, H=1, W=1, C=1024, O=10, KH=1, KW=1, pad=(0, 0, 0, 0)),
    dict(N=1, H=16, W=16, C=32, O=64, KH=3, KW=3),
]


@pytest.mark.parametrize("kw", CONV)
@pytest.mark.parametrize("nhwc", [True, False])
def test_conv2d_descriptor(kw, nhwc):
    wl = w.conv2d_workload(realistic=True, nhwc=nhwc, output_min=-128, **kw)
    outs, d = interp(wl)
    assert_bit_exact(outs[0], oracle_eval(wl)[0], wl.name)
    kinds = [int(o["kind"]) for o in d.ops]
    C, HW = kw["C"], kw["H"] * kw["W"]
    if nhwc or C == 1 or HW == 1:
        assert kinds.count(desc_interp.K_TRANSPOSE) <= (0 if nhwc else 1)
    else:
        assert kinds[0] == desc_interp.K_TRANSPOSE and kinds[1] == desc_interp.K_IGEMM


# Convolutions over a multiple of 16 channels: the LDS-DMA ring kernel addresses the window.
WINDOW_RING = [
    dict(N=2, H=32, W=32, C=64, O=64),                                            # M = 2048: the smallest taken; one tile column
    dict(N=10, H=29, W=31, C=64, O=96, stride=(2, 2), pad=(0, 1, 0, 1)),          # odd frame, stride 2, one-sided padding, ragged M
    dict(N=2, H=40, W=36, C=128, O=160, pad=(1, 1, 1, 1)),                        # two k-tiles per tap, N not a multiple of any tile
    dict(N=1, H=50, W=50, C=64, O=72, KH=5, KW=5, pad=(2, 2, 2, 2)),              # 25 taps; N % 16 != 0: the staged epilogue
    dict(N=2, H=34, W=66, C=64, O=256, KH=1, KW=3, pad=(1, 1, 0, 0)),             # a flat window
    dict(N=8, H=24, W=24, C=192, O=128, KH=3, KW=3, stride=(1, 2), pad=(2, 0, 1, 2)),  # three k-tiles per tap, mixed strides, lopsided pads
    dict(N=8, H=33, W=33, C=64, O=64, KH=1, KW=1, stride=(2, 2), pad=(0, 0, 0, 0)),    # a strided pointwise convolution
    dict(N=3, H=31, W=30, C=80, O=96, pad=(1, 1, 1, 1)),                          # k-tiles straddle taps; K = 720 ends inside the last k-tile
    dict(N=4, H=36, W=34, C=96, O=40, KH=3, KW=3, stride=(2, 1), pad=(0, 2, 1, 0), input_zp=-77),  # K = 864, Kp = 896
    dict(N=2, H=33, W=37, C=144, O=144, KH=2, KW=3, pad=(1, 1, 0, 1), input_zp=55),                # K = 864: taps of 2.25 k-tiles
    dict(N=1, H=60, W=44, C=208, O=64, KH=1, KW=3, pad=(1, 1, 0, 0)),                              # K = 624, Kp = 640
    dict(N=1, H=16, W=16, C=112, O=112, KH=5, KW=5, pad=(2, 2, 2, 2)),                             # few pixels, K = 2800 -> 2816
]

# Fewer channels than a k-tile: the chunks of one k-tile span several taps, up to four window rows (1 x 1 x 16).
WINDOW_RING_FEW_CHANNELS = [
    dict(N=3, H=31, W=30, C=32, O=96, pad=(1, 1, 1, 1)),
    dict(N=4, H=36, W=34, C=16, O=40, KH=3, KW=3, stride=(2, 1), pad=(0, 2, 1, 0), input_zp=-77),
    dict(N=2, H=33, W=37, C=48, O=144, KH=2, KW=3, pad=(1, 1, 0, 1), input_zp=55),
    dict(N=1, H=60, W=44, C=16, O=64, KH=1, KW=3, pad=(1, 1, 0, 0)),
    dict(N=1, H=50, W=50, C=32, O=72, KH=5, KW=5, pad=(2, 2, 2, 2)),
    dict(N=2, H=40, W=40, C=16, O=33, KH=7, KW=7, pad=(3, 3, 3, 3)),
    dict(N=2, H=40, W=40, C=16, O=64, KH=1, KW=2, pad=(0, 1, 0, 0)),
    dict(N=24, H=20, W=20, C=48, O=64, KH=4, KW=1, stride=(2, 2), pad=(0, 0, 1, 2)),
    dict(N=2, H=40, W=40, C=16, O=64, KH=3, KW=1, pad=(0, 0, 1, 1)),
]


def test_conv2d_on_images_smaller_than_one_load():
    """An image of fewer than 16 bytes cannot feed the window-row loader (16-byte loads kept inside the image): such
    convolutions take the gather loader.  (Found by a long run of the random sweep: the launcher refused them.)"""
    for kw in (dict(N=1, H=2, W=6, C=1, O=3, KH=2, KW=1, pad=(0, 0, 1, 0)), dict(N=1, H=11, W=1, C=1, O=15, KH=3, KW=1, pad=(0, 0, 1, 1)),
               dict(N=2, H=1, W=1, C=4, O=3, KH=1, KW=1, pad=(0, 0, 0, 0)), dict(N=1, H=2, W=2, C=3, O=24, KH=2, KW=1, pad=(0, 0, 0, 1)),
               dict(N=1, H=4, W=4, C=1, O=5, KH=3, KW=3)):
        wl = w.conv2d_workload(realistic=True, **kw)
        outs, d = interp(wl)
        assert_bit_exact(outs[0], oracle_eval(wl)[0], wl.name)
        small = kw["N"] * kw["H"] * kw["W"] * kw["C"] < 16
        assert int(d.ops[-1]["loader"]) == (1 if small else 2), (kw, int(d.ops[-1]["loader"]))


def test_dense_k128_records(monkeypatch):
    """A long K with enough 256 x 256 tiles takes the variant with 128-byte k-tiles: K padded to 128, same results."""
    wl = w.fully_connected_workload(3584, 1040, 4096, realistic=True)
    outs, d = interp(wl)
    assert_bit_exact(outs[0], oracle_eval(wl)[0], wl.name)
    assert int(d.ops[0]["variant"]) == 14 and int(d.ops[0]["Kp"]) == 1152
    monkeypatch.setenv("THIP_NO_K128", "1")
    assert int(interp(wl)[1].ops[0]["variant"]) == 4
    monkeypatch.delenv("THIP_NO_K128")
    monkeypatch.setenv("THIP_IGEMM_DENSE_VARIANT", "14")
    for mkn in ((300, 48, 272), (33, 400, 40), (257, 128, 520)):
        wl = w.fully_connected_workload(*mkn, realistic=True)
        outs, d = interp(wl)
        assert_bit_exact(outs[0], oracle_eval(wl)[0], wl.name)
        assert int(d.ops[0]["variant"]) == 14 and int(d.ops[0]["Kp"]) % 128 == 0


def test_dense_tile_choice_by_rounds_of_tiles():
    """K of 513 .. 1024 and more than a tenth of the last round of 256 x 256 tiles idle: two half-size blocks per CU."""
    def variant(M, K, N):
        wl = w.fully_connected_workload(M, K, N, realistic=True, zeros=True)
        return int(desc_interp.Descriptor(wl.program.serialize()).ops[0]["variant"])
    assert variant(100352, 768, 512) == 6      # 784 tiles: 3.06 rounds
    assert variant(100352, 1024, 512) == 6
    assert variant(100352, 1536, 512) == 14    # a long K: 128-byte k-tiles on the largest tile
    assert variant(4096, 768, 4096) == 14      # 256 tiles, one full round: the largest tile, 128-byte k-tiles from K = 576
    assert variant(4096, 528, 4096) == 4       # K would be padded by a quarter: 64-byte k-tiles
    assert variant(6000, 1024, 4096) == 14     # 384 tiles, K = 1024: no gain measured
    assert variant(6000, 896, 4096) == 6


def test_conv2d_window_loader_records():
    """A multiple of 16 channels: the record asks for the ring kernel's window addressing (loader 3, a page of
    zero-point bytes as its table, K rounded up to whole k-tiles); other channel counts or the switch keep the gather
    loader."""
    import os
    for kw in WINDOW_RING:
        wl = w.conv2d_workload(realistic=True, **kw)
        outs, d = interp(wl)
        assert_bit_exact(outs[0], oracle_eval(wl)[0], wl.name)
        assert [(int(o["kind"]), int(o["loader"])) for o in d.ops] == [(desc_interp.K_IGEMM, 3)], wl.name
        bk = 128 if int(d.ops[0]["variant"]) == 14 else 64
        assert int(d.ops[0]["Kp"]) == -(-int(d.ops[0]["K"]) // bk) * bk
    for kw in (dict(N=2, H=32, W=32, C=72, O=64), dict(N=2, H=32, W=32, C=40, O=64)):
        d = interp(w.conv2d_workload(realistic=True, **kw))[1]
        assert int(d.ops[0]["loader"]) == 1, kw
    # small convolutions take the 64 x 64 tile (up to 512 of them)
    for kw, variant in ((dict(N=1, H=32, W=32, C=64, O=64), 7), (dict(N=1, H=7, W=7, C=160, O=160), 7), (dict(N=1, H=28, W=28, C=32, O=32), 7),
                        (dict(N=16, H=14, W=14, C=512, O=512), 7), (dict(N=32, H=14, W=14, C=512, O=512), 5),
                        (dict(N=2, H=32, W=32, C=64, O=16), 7), (dict(N=1, H=28, W=28, C=64, O=8), 7), (dict(N=48, H=32, W=32, C=16, O=24), 10), (dict(N=48, H=32, W=32, C=16, O=40), 9)):
        wl = w.conv2d_workload(realistic=True, **kw)
        outs, d = interp(wl)
        assert_bit_exact(outs[0], oracle_eval(wl)[0], wl.name)
        assert (int(d.ops[0]["loader"]), int(d.ops[0]["variant"])) == (3, variant), kw
    os.environ["THIP_NO_WINDOW_RING"] = "1"
    try:
        assert int(interp(w.conv2d_workload(realistic=True, **WINDOW_RING[0]))[1].ops[0]["loader"]) == 1
    finally:
        del os.environ["THIP_NO_WINDOW_RING"]


@pytest.mark.parametrize("variant", [None, 14])
def test_conv2d_window_loader_few_channels(variant, monkeypatch):
    """16, 32 and 48 channels on the window loader: several taps per k-tile."""
    if variant is not None:
        monkeypatch.setenv("THIP_WINDOW_VARIANT", str(variant))
    for kw in WINDOW_RING_FEW_CHANNELS:
        wl = w.conv2d_workload(realistic=True, **kw)
        outs, d = interp(wl)
        assert_bit_exact(outs[0], oracle_eval(wl)[0], wl.name)
        assert [(int(o["kind"]), int(o["loader"])) for o in d.ops] == [(desc_interp.K_IGEMM, 3)], wl.name


@pytest.mark.parametrize("kw", [
    dict(N=1, H=6, W=42, C=16), dict(N=1, H=6, W=6, C=2, pad=(0, 0, 0, 0)), dict(N=1, H=13, W=15, C=8, stride=(1, 1), pad=(1, 1, 1, 1)),
    dict(N=1, H=27, W=27, C=128, KH=4, KW=4, stride=(2, 2), pad=(1, 2, 1, 2)), dict(N=2, H=21, W=21, C=5, stride=(2, 2), pad=(1, 1, 1, 1)),
])
@pytest.mark.parametrize("nhwc", [True, False])
def test_depthwise_descriptor(kw, nhwc):
    wl = w.depthwise_workload(nhwc=nhwc, **kw)
    outs, _ = interp(wl)
    assert_bit_exact(outs[0], oracle_eval(wl)[0], wl.name)


@pytest.mark.parametrize("mkn", [(1, 1, 1), (1, 61, 1991), (4, 1024, 1024), (1, 2000, 97), (16, 3, 7), (17, 128, 70), (130, 700, 500)])
def test_fully_connected_descriptor(mkn):
    wl = w.fully_connected_workload(*mkn, realistic=True)
    outs, d = interp(wl)
    assert_bit_exact(outs[0], oracle_eval(wl)[0], wl.name)
    M, K, _ = mkn
    want_kind = desc_interp.K_FC_SKINNY if (M <= 16 and K % 16 == 0) else desc_interp.K_IGEMM
    assert int(d.ops[0]["kind"]) == want_kind


# int8 torq_hl.matmul.  The first five are the shapes of the reference's own fixtures:
# tests/testdata/tosa_ops/matmul-in-int8-out-int16-{1024x128x1024,64x128x2048}.mlir and
# tests/testdata/linalg_ops/{matmul-in-int8-out-int16-noalign,batch-matmul-in-int8-out-int16,matvec-in-int8-out-int16}.mlir
# (12x56x168 has K % 16 != 0; the matrix-vector product is N = 1).  Then: batch broadcast on either side, constant
# and run-time input2, every result type, a real rescale, ragged K and N.
MATMUL = [
    dict(B=1, M=1024, K=128, N=1024),
    dict(B=1, M=64, K=128, N=2048),
    dict(B=1, M=12, K=56, N=168, batch1=False, batch2=False),
    dict(B=1, M=64, K=128, N=256),
    dict(B=1, M=128, K=64, N=1, batch1=False, batch2=False),
    dict(B=3, M=20, K=64, N=48, batch1=False),
    dict(B=3, M=20, K=64, N=48, batch2=False),
    dict(B=3, M=20, K=64, N=48, batch1=False, constant_rhs=True),
    dict(B=2, M=33, K=96, N=40, batch2=False, constant_rhs=True),
    dict(B=2, M=33, K=96, N=40, constant_rhs=True, out_dtype=np.int32),
    dict(B=2, M=9, K=61, N=37, out_dtype=np.int32),
    dict(B=2, M=9, K=61, N=37, constant_rhs=True, out_dtype=np.int8, bias=-77, scale=(1 << 30) + 12345, shift=41, output_zp=3),
    dict(B=1, M=300, K=80, N=130, out_dtype=np.int8, bias=1234, scale=(1 << 30) + 999, shift=42, output_zp=-5, clamp=(-100, 90)),
    dict(B=2, M=5, K=7, N=3, bias=5, scale=3, shift=1),
]


def matmul_id(kw):
    return "-".join("%s%s" % (k[:2], getattr(v, "__name__", v)) for k, v in kw.items())


@pytest.mark.parametrize("kw", MATMUL, ids=matmul_id)
def test_matmul_descriptor(kw):
    wl = w.matmul_workload(**kw)
    outs, d = interp(wl)
    want = oracle_eval(wl)[0]
    assert_bit_exact(outs[0], want, wl.name)
    kinds = [int(o["kind"]) for o in d.ops]
    Bb = kw["B"] if kw.get("batch2", True) else 1
    if kw.get("constant_rhs"):
        assert kinds == [desc_interp.K_IGEMM] * Bb  # one record per weight matrix; a broadcast input2 takes all rows at once
    else:
        assert kinds == [desc_interp.K_TRANSPOSE] * Bb + [desc_interp.K_IGEMM] * kw["B"]
        assert all(int(o["TP"]) == int(d.ops[-1]["Kp"]) for o in d.ops[:Bb])  # transposed into zero-padded rows of Kp
    if kw.get("out_dtype", np.int16) == np.int16 and kw["K"] >= 64 and "scale" not in kw:
        assert (want == 32767).any() or (want == -32768).any() or kw["K"] < 128  # int16 results of a long K saturate: the clamp is exercised


@pytest.mark.parametrize("kw", [dict(H=8, W=8, C=4), dict(H=32, W=32, C=64, kernel=(3, 3), pad=(1, 1, 1, 1)), dict(H=10, W=10, C=4, kernel=(5, 5), stride=(1, 1)),
                                dict(H=10, W=10, C=4, kernel=(1, 3), stride=(1, 3), pad=(0, 2, 0, 0), input_zp=-7)])
@pytest.mark.parametrize("nhwc", [True, False])
def test_maxpool_descriptor(kw, nhwc):
    wl = w.maxpool_workload(nhwc=nhwc, **kw)
    outs, _ = interp(wl)
    assert_bit_exact(outs[0], oracle_eval(wl)[0], wl.name)


def test_avgpool_and_add_descriptor():
    for wl in (w.avgpool_workload(N=2, C=128), w.avgpool_workload(N=1, H=12, W=8, C=37), w.add_workload(), w.add_workload(N=1, H=4, W=4, C=1)):
        outs, _ = interp(wl)
        assert_bit_exact(outs[0], oracle_eval(wl)[0], wl.name)


def _chain_program(nchw_bindings):
    """conv(1x1 expand) -> depthwise -> conv(1x1 project) -> add residual -> transpose -> avg_pool -> fc,
    all declared N,C,H,W like the reference emits them."""
    rng = np.random.default_rng(77)
    N, C, H, W, E = 2, 16, 10, 10, 48
    x = rng.integers(-128, 128, size=(N, C, H, W)).astype(np.int8)
    prm = {}

    def conv_params(O, wshape, zp):
        wt = rng.integers(-127, 128, size=wshape).astype(np.int8)
        mult, shift = w.random_requant(rng, O, True)
        sb, sf = w.derive_scale_bias(mult, (shift - 3).astype(np.int8), rng.integers(-2000, 2000, size=O), wt, zp)
        return wt, sb, sf

    prm["w1"], prm["sb1"], prm["sf1"] = conv_params(E, (E, C, 1, 1), -3)
    prm["wd"], prm["sbd"], prm["sfd"] = conv_params(E, (E, 1, 3, 3), 2)
    prm["w2"], prm["sb2"], prm["sf2"] = conv_params(C, (C, E, 1, 1), -1)
    prm["aw"], prm["asb"], prm["asf"] = w.add_params(0.6, 0.9, -3, 4)
    prm["psb"] = np.array([-(H * W * 1), (1 << 20) // (H * W)], dtype=np.int32)
    prm["wf"], prm["sbf"], prm["sff"] = conv_params(10, (10, C), 0)

    p = Program()
    xin = p.binding(0, x.shape)
    t1 = p.conv2d(xin, prm["w1"], prm["sb1"], input_zp=-3, output_zp=2, output_min=-128, output_max=127, shift_factor=prm["sf1"], pad=(0, 0, 0, 0), stride=(1, 1))
    t2 = p.depthwise_conv2d(t1, prm["wd"], prm["sbd"], input_zp=2, output_zp=-1, output_min=-128, output_max=127, shift_factor=prm["sfd"], pad=(1, 1, 1, 1), stride=(1, 1))
    t3 = p.conv2d(t2, prm["w2"], prm["sb2"], input_zp=-1, output_zp=4, output_min=-128, output_max=127, shift_factor=prm["sf2"], pad=(0, 0, 0, 0), stride=(1, 1))
    t4 = p.add(xin, t3, prm["aw"], prm["asb"], output_zp=1, output_min=-128, output_max=127, shift_factor=prm["asf"])
    t5 = p.transpose(t4, (0, 2, 3, 1))
    t6 = p.avg_pool2d(t5, np.array([1], dtype=np.int8), prm["psb"], input_zp=1, output_zp=0, output_min=-128, output_max=127, shift_factor=20)
    out = p.binding(1, (N, 10))
    p.fully_connected(t6, prm["wf"], prm["sbf"], init=out, output_zp=3, output_min=-128, output_max=127, shift_factor=prm["sff"])
    aux = p.binding(2, (N, C, H, W))  # also export the residual sum, N,C,H,W
    p.add(xin, t3, prm["aw"], prm["asb"], init=aux, output_zp=1, output_min=-128, output_max=127, shift_factor=prm["asf"])

    # oracle, literal N,C,H,W
    o1 = orc.conv2d(x, prm["w1"], prm["sb1"], input_zp=-3, output_zp=2, output_min=-128, output_max=127, shift_factor=prm["sf1"], pad=(0, 0, 0, 0), stride=(1, 1))
    o2 = orc.depthwise_conv2d(o1, prm["wd"], prm["sbd"], input_zp=2, output_zp=-1, output_min=-128, output_max=127, shift_factor=prm["sfd"], pad=(1, 1, 1, 1), stride=(1, 1))
    o3 = orc.conv2d(o2, prm["w2"], prm["sb2"], input_zp=-1, output_zp=4, output_min=-128, output_max=127, shift_factor=prm["sf2"], pad=(0, 0, 0, 0), stride=(1, 1))
    o4 = orc.add(x, o3, prm["aw"], prm["asb"], output_zp=1, output_min=-128, output_max=127, shift_factor=prm["asf"])
    o5 = np.ascontiguousarray(o4.transpose(0, 2, 3, 1))
    o6 = orc.avg_pool2d(o5, prm["psb"], output_zp=0, output_min=-128, output_max=127, shift_factor=20)
    o7 = orc.fully_connected(o6.reshape(N, C), prm["wf"], prm["sbf"], output_zp=3, output_min=-128, output_max=127, shift_factor=prm["sff"])
    return p, x, o7, o4


def test_multi_op_program_keeps_intermediates_nhwc():
    p, x, want_fc, want_sum = _chain_program(True)
    blob = p.serialize()
    out = np.zeros(want_fc.shape, dtype=np.int8)
    aux = np.zeros(want_sum.shape, dtype=np.int8)
    d = desc_interp.run(blob, [x, out, aux])
    assert_bit_exact(out, want_fc, "chain fc")
    assert_bit_exact(aux, want_sum, "chain residual")
    kinds = [int(o["kind"]) for o in d.ops]
    # one transpose brings the N,C,H,W binding in (shared by conv and both adds would be ideal; each
    # consumer of the literal binding converts it), one takes the exported sum out; none in between.
    first_igemm = kinds.index(desc_interp.K_IGEMM)
    between = kinds[first_igemm:kinds.index(desc_interp.K_AVGPOOL)]
    assert desc_interp.K_TRANSPOSE not in [k for k in between if k != desc_interp.K_ADD][0:3]
    assert kinds[-1] == desc_interp.K_TRANSPOSE


def test_rejects_what_the_path_does_not_cover():
    def expect(code, build):
        p = Program()
        with pytest.raises(ThipError) as e:
            build(p)
            p.serialize()
        assert e.value.code == code, e.value

    x8 = np.zeros((4, 3, 3, 3), dtype=np.int8)
    sb = np.zeros(8, dtype=np.int32)
    common = dict(input_zp=0, output_zp=0, output_min=-128, output_max=127, shift_factor=4, pad=(0, 0, 0, 0), stride=(1, 1))
    expect(runtime.UNIMPLEMENTED, lambda p: p.conv2d(p.binding(0, (1, 3, 8, 8)), x8, sb, init=p.binding(1, (1, 4, 6, 6)), groups=2, **common))
    expect(runtime.UNIMPLEMENTED, lambda p: p.conv2d(p.binding(0, (1, 3, 8, 8)), x8, sb, init=p.binding(1, (1, 4, 6, 6)), dilation=(2, 2), **common))
    expect(runtime.UNIMPLEMENTED, lambda p: p.conv2d(p.binding(0, (1, 3, 8, 8)), x8, sb, init=p.binding(1, (1, 4, 6, 6)), weight_zp=1, **common))
    expect(runtime.INVALID_ARGUMENT, lambda p: p.conv2d(p.binding(0, (1, 5, 8, 8)), x8, sb, init=p.binding(1, (1, 4, 6, 6)), **common))
    expect(runtime.INVALID_ARGUMENT, lambda p: p.conv2d(p.binding(0, (1, 3, 8, 8)), x8, sb, init=p.binding(1, (1, 4, 7, 6)), **common))
    bad = dict(common, shift_factor=64)
    expect(runtime.INVALID_ARGUMENT, lambda p: p.conv2d(p.binding(0, (1, 3, 8, 8)), x8, sb, init=p.binding(1, (1, 4, 6, 6)), **bad))
    bad = dict(common, output_zp=40000)
    expect(runtime.INVALID_ARGUMENT, lambda p: p.conv2d(p.binding(0, (1, 3, 8, 8)), x8, sb, init=p.binding(1, (1, 4, 6, 6)), **bad))
    bad = dict(common, output_max=300)
    expect(runtime.INVALID_ARGUMENT, lambda p: p.conv2d(p.binding(0, (1, 3, 8, 8)), x8, sb, init=p.binding(1, (1, 4, 6, 6)), **bad))
    # weights must be compile-time constants
    expect(runtime.UNIMPLEMENTED, lambda p: p.conv2d(p.binding(0, (1, 3, 8, 8)), p.binding(2, (4, 3, 3, 3)), sb, init=p.binding(1, (1, 4, 6, 6)), **common))
    # reading an intermediate that nothing wrote
    expect(runtime.FAILED_PRECONDITION, lambda p: p.maxpool2d(p.tensor((1, 3, 8, 8)), input_zp=-128, output_min=-128, output_max=127, stride=(2, 2), pad=(0, 0, 0, 0), kernel=(2, 2), init=p.binding(0, (1, 3, 4, 4))))
    expect(runtime.INVALID_ARGUMENT, lambda p: None)  # empty program


def test_descriptor_header_and_format():
    wl = w.add_workload(N=1, H=2, W=2, C=4)
    blob = wl.program.serialize()
    fmt, size = runtime.infer_format(blob)
    assert fmt == "thip-gfx950" and size == len(blob)
    d = desc_interp.Descriptor(blob)
    assert d.header["version"] == runtime.lib().thip_descriptor_version() and d.header["arch"] == 950
    assert [int(b["flags"]) for b in d.bindings] == [1, 1, 2]  # read, read, written
    for mutate, code in [((0, b"XXXX"), runtime.INVALID_ARGUMENT), ((4, (99).to_bytes(4, "little")), runtime.UNAVAILABLE),
                         ((8, (942).to_bytes(4, "little")), runtime.UNAVAILABLE)]:
        bad = bytearray(blob)
        bad[mutate[0]:mutate[0] + 4] = mutate[1]
        with pytest.raises(ThipError) as e:
            runtime.infer_format(bytes(bad))
        assert e.value.code == code
    with pytest.raises(ThipError) as e:
        runtime.infer_format(blob[:40])
    assert e.value.code == runtime.INVALID_ARGUMENT
    with pytest.raises(ThipError) as e:
        runtime.infer_format(blob[:-1])
    assert e.value.code == runtime.INVALID_ARGUMENT


def _padded_chain(nhwc):
    """conv 1x1 (16->24) -> depthwise 3x3 -> maxpool 2x2 -> conv 3x3 (24->24) -> add -> conv 1x1 (24->40):
    every intermediate has 24 channels, which the emitter stores as 32."""
    rng = np.random.default_rng(5)
    N, C, H, W, B = 2, 16, 12, 12, 24
    x = rng.integers(-128, 128, size=(N, H, W, C) if nhwc else (N, C, H, W)).astype(np.int8)
    lay = orc.NHWC if nhwc else orc.NCHW
    rq = dict(output_min=-128, output_max=127)

    def params(O, wshape, zp):
        wt = rng.integers(-127, 128, size=wshape).astype(np.int8)
        mult, shift = w.random_requant(rng, O, True)
        sb, sf = w.derive_scale_bias(mult, (shift - 3).astype(np.int8), rng.integers(-2000, 2000, size=O), wt, zp)
        return wt, sb, sf

    w1, sb1, sf1 = params(B, (B, C, 1, 1), -3)
    wd, sbd, sfd = params(B, (B, 1, 3, 3), 2)
    w3, sb3, sf3 = params(B, (B, B, 3, 3), 5)
    aw, asb, asf = w.add_params(0.7, 0.8, 5, -6)
    w5, sb5, sf5 = params(40, (40, B, 1, 1), 1)
    p = Program()
    xin = p.binding(0, x.shape)
    kw = dict(nhwc_input=nhwc)
    t1 = p.conv2d(xin, w1, sb1, input_zp=-3, output_zp=2, shift_factor=sf1, pad=(0, 0, 0, 0), stride=(1, 1), **rq, **kw)
    t2 = p.depthwise_conv2d(t1, wd, sbd, input_zp=2, output_zp=5, shift_factor=sfd, pad=(1, 1, 1, 1), stride=(1, 1), **rq, **kw)
    t3 = p.maxpool2d(t2, input_zp=5, stride=(2, 2), pad=(0, 0, 0, 0), kernel=(2, 2), **rq, **kw)
    t4 = p.conv2d(t3, w3, sb3, input_zp=5, output_zp=-6, shift_factor=sf3, pad=(1, 1, 1, 1), stride=(1, 1), **rq, **kw)
    t5 = p.add(t3, t4, aw, asb, output_zp=1, shift_factor=asf, **rq)
    oshape = (N, H // 2, W // 2, 40) if nhwc else (N, 40, H // 2, W // 2)
    p.conv2d(t5, w5, sb5, init=p.binding(1, oshape), input_zp=1, output_zp=0, shift_factor=sf5, pad=(0, 0, 0, 0), stride=(1, 1), **rq, **kw)

    o1 = orc.conv2d(x, w1, sb1, input_zp=-3, output_zp=2, shift_factor=sf1, pad=(0, 0, 0, 0), stride=(1, 1), layout=lay, **rq)
    o2 = orc.depthwise_conv2d(o1, wd, sbd, input_zp=2, output_zp=5, shift_factor=sfd, pad=(1, 1, 1, 1), stride=(1, 1), layout=lay, **rq)
    o3 = orc.maxpool2d(o2, input_zp=5, stride=(2, 2), pad=(0, 0, 0, 0), kernel=(2, 2), layout=lay, **rq)
    o4 = orc.conv2d(o3, w3, sb3, input_zp=5, output_zp=-6, shift_factor=sf3, pad=(1, 1, 1, 1), stride=(1, 1), layout=lay, **rq)
    o5 = orc.add(o3, o4, aw, asb, output_zp=1, shift_factor=asf, **rq)
    o6 = orc.conv2d(o5, w5, sb5, input_zp=1, output_zp=0, shift_factor=sf5, pad=(0, 0, 0, 0), stride=(1, 1), layout=lay, **rq)
    return p, x, o6


@pytest.mark.parametrize("nhwc", [True, False])
@pytest.mark.parametrize("pad_off", [False, True])
def test_channel_padding_of_intermediates(nhwc, pad_off, monkeypatch):
    if pad_off:
        monkeypatch.setenv("THIP_NO_CHANNEL_PAD", "1")
    p, x, want = _padded_chain(nhwc)
    blob = p.serialize()
    out = np.zeros(want.shape, dtype=np.int8)
    d = desc_interp.run(blob, [x, out])
    assert_bit_exact(out, want, "padded chain")
    ops = [o for o in d.ops if int(o["kind"]) != desc_interp.K_TRANSPOSE]
    c = 24 if pad_off else 32
    assert [int(o["kind"]) for o in ops] == [desc_interp.K_IGEMM, desc_interp.K_DW, desc_interp.K_MAXPOOL,
                                             desc_interp.K_IGEMM, desc_interp.K_ADD, desc_interp.K_IGEMM]
    assert int(ops[0]["Nn"]) == c and int(ops[1]["C"]) == c and int(ops[2]["C"]) == c
    assert int(ops[3]["C"]) == c and int(ops[3]["Nn"]) == c and int(ops[3]["gran"]) == (8 if pad_off else 16)
    assert int(ops[4]["C"]) == 2 * 6 * 6 * c
    assert int(ops[5]["K"]) == c and int(ops[5]["loader"]) == (1 if pad_off else 0) and int(ops[5]["Nn"]) == 40
    assert int(ops[1]["variant"]) == (0 if pad_off else 1)


def test_channel_padding_stops_at_ops_that_read_declared_order():
    """A 24-channel tensor that feeds avg_pool2d (or leaves through a binding) is stored as declared."""
    rng = np.random.default_rng(6)
    N, H, W, C, B = 2, 5, 5, 16, 24
    x = rng.integers(-128, 128, size=(N, H, W, C)).astype(np.int8)
    wt = rng.integers(-127, 128, size=(B, C, 1, 1)).astype(np.int8)
    mult, shift = w.random_requant(rng, B, True)
    sb, sf = w.derive_scale_bias(mult, (shift - 3).astype(np.int8), rng.integers(-100, 100, size=B), wt, 0)
    psb = np.array([0, (1 << 20) // (H * W)], dtype=np.int32)
    rq = dict(output_min=-128, output_max=127)
    p = Program()
    t1 = p.conv2d(p.binding(0, x.shape), wt, sb, input_zp=0, output_zp=0, shift_factor=sf, pad=(0, 0, 0, 0), stride=(1, 1), nhwc_input=True, **rq)
    p.avg_pool2d(t1, np.array([1], dtype=np.int8), psb, init=p.binding(1, (N, 1, 1, B)), input_zp=0, output_zp=0, shift_factor=20, **rq)
    o1 = orc.conv2d(x, wt, sb, input_zp=0, output_zp=0, shift_factor=sf, pad=(0, 0, 0, 0), stride=(1, 1), layout=orc.NHWC, **rq)
    want = orc.avg_pool2d(o1, psb, output_zp=0, shift_factor=20, **rq)
    out = np.zeros(want.shape, dtype=np.int8)
    d = desc_interp.run(p.serialize(), [x, out])
    assert_bit_exact(out, want, "conv -> avg_pool2d")
    assert int(d.ops[0]["Nn"]) == B and int(d.ops[1]["C"]) == B


def test_pre_shift_identity_and_emitter_bound():
    """A shift below 33 with (acc + bias) << (33 - shift) still inside 32 bits equals the shift-33 form the
    kernels evaluate with a 32-bit multiply-high; the emitter sets pre_shift only under that bound."""
    rng = np.random.default_rng(9)
    for shift in range(3, 33):
        pre = 33 - shift
        lim = 1 << (31 - pre)
        t0 = rng.integers(-lim + 1, lim, size=20000, dtype=np.int64)
        t0[:4] = [-lim + 1, lim - 1, 0, -1]
        scale = rng.integers(-(1 << 31), 1 << 31, size=t0.size, dtype=np.int64)
        scale[:4] = [(1 << 31) - 1, -(1 << 31), (1 << 31) - 1, -(1 << 31)]
        want = [(int(a) * int(b) + (1 << (shift - 1))) >> shift for a, b in zip(t0, scale)]
        got = [((((int(a) << pre) * int(b)) >> 32) + 1) >> 1 for a, b in zip(t0, scale)]
        assert want == got, shift
    # emitter: small-K op with shift 24 gets pre_shift 9; a large bias or a tiny shift gets none
    wl = w.fully_connected_workload(64, 64, 32, shift=24)
    assert int(desc_interp.Descriptor(wl.program.serialize()).ops[0]["pre_shift"]) == 9
    # K too large for the bound: acc + bias is clamped instead, to a range where every channel is saturated
    wl = w.fully_connected_workload(64, 4096, 32, shift=24)
    op = desc_interp.Descriptor(wl.program.serialize()).ops[0]
    assert int(op["pre_shift"]) == 9 and int(op["t0_clamp"]) == (1 << 22) - 1
    out = np.zeros(wl.outputs[0][0], dtype=wl.outputs[0][1])
    desc_interp.run(wl.program.serialize(), list(wl.inputs) + [out])
    assert_bit_exact(out, oracle_eval(wl)[0], "clamped pre-shift")
    wl = w.fully_connected_workload(64, 64, 32, shift=2)
    assert int(desc_interp.Descriptor(wl.program.serialize()).ops[0]["pre_shift"]) == 0


@pytest.mark.parametrize("shift,scale_bits", [(10, 14), (10, 9), (6, 31), (20, 22), (3, 4), (32, 30)])
def test_t0_clamp_keeps_results(shift, scale_bits):
    """Small shifts with scales of either sign (and zero): where the emitter clamps acc + bias the 32-bit tail
    still gives the oracle's bytes, in range and saturated; where a channel would not be saturated it must not clamp."""
    rng = np.random.default_rng(shift * 100 + scale_bits)
    M, K, N = 40, 256, 48
    x = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    wt = rng.integers(-127, 128, size=(N, K)).astype(np.int8)
    wt[:, K // 2:] = 0
    wt[::3] = rng.integers(-2, 3, size=wt[::3].shape)  # some channels with small accumulators: unsaturated results
    sb = np.zeros(2 * N, dtype=np.int32)
    sb[0::2] = rng.integers(-3000, 3000, size=N)
    lim = (1 << scale_bits) - 1
    sb[1::2] = rng.integers(-lim, lim, size=N, endpoint=True)
    sb[1] = 0
    p = Program()
    out_b = p.binding(1, (M, N))
    p.fully_connected(p.binding(0, (M, K)), wt, sb, init=out_b, output_zp=-5, output_min=-128, output_max=127, shift_factor=shift)
    want = orc.fully_connected(x, wt, sb, output_zp=-5, output_min=-128, output_max=127, shift_factor=shift)
    out = np.zeros((M, N), dtype=np.int8)
    d = desc_interp.run(p.serialize(), [x, out])
    assert_bit_exact(out, want, "fc shift %d" % shift)
    op = d.ops[0]
    if int(op["t0_clamp"]):
        assert int(op["pre_shift"]) == 33 - shift
    assert scale_bits > 24 or len(np.unique(want)) > 3  # not everything saturated


# ---- residual add folded into the pointwise convolution --------------------------------------------------
@pytest.mark.parametrize("kw", [dict(), dict(other_first=True), dict(N=1, H=65, W=66, C=32, O=16), dict(N=3, H=40, W=40, C=144, O=48, other_first=True),
                                dict(N=1, H=8, W=8), dict(N=1, H=14, W=14, C=384, O=64, other_first=True), dict(N=2, H=7, W=7, C=960, O=160)])
def test_residual_add_folds_into_the_streaming_convolution(kw):
    """Many pixels: the pixel-streaming kernel; few: the 64x64 dense tile with its in-register epilogue."""
    wl = w.pointwise_add_workload(**kw)
    outs = [np.zeros(s, dtype=dt) for s, dt in wl.outputs]
    d = desc_interp.run(wl.program.serialize(), list(wl.inputs) + outs)
    assert_bit_exact(outs[0], oracle_eval(wl)[0], wl.name)
    assert [int(o["kind"]) for o in d.ops] == [desc_interp.K_IGEMM] and int(d.ops[0]["in1"]["space"]) != 0
    assert all(int(t["size"]) == 0 for t in d.temps)  # the convolution's own result is never materialised


def test_residual_add_stays_apart_when_it_must(monkeypatch):
    def kinds(p):
        return [int(o["kind"]) for o in desc_interp.Descriptor(p.serialize()).ops]

    monkeypatch.setenv("THIP_NO_ADD_FUSION", "1")
    assert kinds(w.pointwise_add_workload().program) == [desc_interp.K_IGEMM, desc_interp.K_ADD]
    monkeypatch.delenv("THIP_NO_ADD_FUSION")
    # output channels that are not a multiple of 16: neither kernel that can add a residual takes them
    assert kinds(w.pointwise_add_workload(O=24).program) == [desc_interp.K_IGEMM, desc_interp.K_ADD]
    # the convolution's result has a second reader
    wl = w.pointwise_add_workload()
    wp, sbp, pa = wl.attrs["pw"]
    aw, asb, aa = wl.attrs["add"]
    p = Program()
    t = p.conv2d(p.binding(0, wl.inputs[0].shape), wp, sbp, nhwc_input=True, **pa)
    s1 = p.add(t, p.binding(1, wl.inputs[1].shape), aw, asb, init=p.binding(2, wl.inputs[1].shape), **aa)
    p.add(t, s1, aw, asb, init=p.binding(3, wl.inputs[1].shape), **aa)
    assert kinds(p) == [desc_interp.K_IGEMM, desc_interp.K_ADD, desc_interp.K_ADD]


def test_descriptor_in_the_terms_of_the_reference_schema():
    """The blob read back as the reference's ExecutableDef concepts (runtime/schemas/torq_executable_def.fbs:13-48,168-197):
    executable name, runtime version / hardware id gates, the binding table {id, address, offset, size, is_read_only,
    is_write_only}, the constant segments."""
    p, x, want_fc, want_sum = _chain_program(True)
    p.set_name("main_dispatch_0_conv2d")
    blob = p.serialize()
    info, bindings, segments = runtime.describe_blob(blob)
    d = desc_interp.Descriptor(blob)
    assert info["executable_name"] == "main_dispatch_0_conv2d" and info["runtime_version"] == 2 and info["hw_id"] == 950
    assert info["action_count"] == len(d.ops) and info["total_size"] == len(blob)
    assert info["intermediate_count"] == len(d.temps) and info["intermediate_bytes"] == int(d.temps["size"].sum())
    # binding 0 is the input (read only), bindings 1 and 2 are results (write only); sizes are the bytes touched
    assert [b["id"] for b in bindings] == [0, 1, 2]
    assert [(b["is_read_only"], b["is_write_only"]) for b in bindings] == [(True, False), (False, True), (False, True)]
    assert [b["size"] for b in bindings] == [x.nbytes, want_fc.nbytes, want_sum.nbytes]
    assert all(b["address"] == 0 and b["offset"] == 0 and b["is_used"] for b in bindings)
    # segments: what create uploads once; they tile the data region without overlap, 256-byte aligned
    assert len(segments) == len(d.consts) and segments
    end = 0
    for s, c in zip(segments, d.consts):
        assert s["address"] == int(c["offset"]) and s["size"] == int(c["size"]) and s["address"] % 256 == 0 and s["address"] >= end
        end = s["address"] + s["size"]
    assert all(s["data"] == bytes(d.const_bytes(i)) for i, s in enumerate(segments))
    # a binding that is both read and written is neither read-only nor write-only
    q = Program()
    a = q.binding(0, (1, 8, 8, 16))
    q.maxpool2d(a, input_zp=-128, output_min=-128, output_max=127, stride=(1, 1), pad=(0, 0, 0, 0), kernel=(1, 1), init=q.binding(1, (1, 8, 8, 16)), nhwc_input=True)
    q.maxpool2d(q.binding(1, (1, 8, 8, 16)), input_zp=-128, output_min=-128, output_max=127, stride=(1, 1), pad=(0, 0, 0, 0), kernel=(1, 1),
                init=q.binding(2, (1, 8, 8, 16)), nhwc_input=True)
    _, b2, _ = runtime.describe_blob(q.serialize())
    assert (b2[1]["is_read_only"], b2[1]["is_write_only"]) == (False, False)
    # names that would not survive as a directory or a CSV column are refused
    for bad in ["", "a/b", "x,y", "..", "n" * 64]:
        with pytest.raises(ThipError):
            Program().set_name(bad)
