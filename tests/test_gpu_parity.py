"""Parity of the HIP kernels with the CPU oracle, through the C-ABI, on a real gfx950.

Bit-exact: every op is integer.  Each case is printed (and flushed) before it touches the GPU so
that a fault names its case.
"""
import sys

import numpy as np
import pytest

from helpers import assert_bit_exact, families, oracle_eval, oracle_network, run_on_gpu
from test_emitter import CONV, MATMUL, WINDOW_RING, WINDOW_RING_FEW_CHANNELS, _chain_program, _padded_chain, matmul_id
from torq_compiler_amd import Executable, ThipError, runtime, workloads as w

pytestmark = pytest.mark.gpu


def announce(*what):
    print("[gpu-case]", *what, flush=True)
    sys.stdout.flush()


def check(device, wl, via="host", kernel=None):
    announce(wl.name, "via", via)
    got, kernels = run_on_gpu(device, wl, via=via)
    want = oracle_eval(wl)
    assert_bit_exact(got[0], want[0], wl.name)
    if kernel is not None:
        # `kernel` names what rocprof would show for the op: a whole instantiation ("name<args>") must match exactly,
        # a bare name must be the name in front of the template arguments
        if "<" in kernel:
            assert kernel in kernels, (kernels, kernel)
        else:
            assert kernel in families(kernels), (kernels, kernel)
    return kernels


# ---- conv2d ---------------------------------------------------------------------------------
def test_conv2d_config0_literal(device):
    """benchmark configuration 0 with its literal (saturating) requant ranges."""
    check(device, w.conv2d_workload(), kernel="igemm_dense_conv_i8")


def test_conv2d_config0_realistic(device):
    check(device, w.conv2d_workload(realistic=True), via="device", kernel="igemm_dense_conv_i8")


def test_conv2d_config0_nchw_boundary(device):
    """Same op with the reference's literal N,C,H,W boundary: transposes at the bindings."""
    kernels = check(device, w.conv2d_workload(realistic=True, nhwc=False))
    assert kernels[0] == "transpose_i8<1>" and kernels[-1] == "transpose_i8<1>"


@pytest.mark.parametrize("kw", CONV)
@pytest.mark.parametrize("nhwc", [True, False])
def test_conv2d_geometries(device, kw, nhwc):
    check(device, w.conv2d_workload(realistic=True, nhwc=nhwc, output_min=-128, **kw))


@pytest.mark.parametrize("variant", [0, 1, 2, 3])
def test_conv2d_every_tile_variant(device, variant, monkeypatch):
    monkeypatch.setenv("THIP_IGEMM_VARIANT", str(variant))
    k = check(device, w.conv2d_workload(N=2, H=28, W=28, C=24, O=96, realistic=True))  # 24 channels: the gather kernel
    assert runtime.lib()  # the variant is baked into the descriptor at serialize time
    names = ["igemm_i8<128,128,64,", "igemm_i8<256,256,64,", "igemm_i8<64,64,64,", "igemm_i8<256,128,64,"]
    assert k[0].startswith(names[variant]), k
    check(device, w.conv2d_workload(N=1, H=15, W=17, C=24, O=40, KH=1, KW=1, pad=(0, 0, 0, 0), realistic=True))
    check(device, w.fully_connected_workload(300, 192, 520, realistic=True))


@pytest.mark.parametrize("kw", WINDOW_RING, ids=lambda kw: "x".join(str(kw[k]) for k in ("N", "H", "W", "C", "O")))
def test_conv2d_window_ring(device, kw):
    """Convolutions over a multiple of 16 channels, 64 or more: the LDS-DMA ring kernel addresses the window itself."""
    k = check(device, w.conv2d_workload(realistic=True, **kw), via="device")
    assert families(k) == ["igemm_dense_conv_i8"], k
    k = check(device, w.conv2d_workload(realistic=False, nhwc=False, **kw))  # the literal requant range, N,C,H,W bindings
    assert "igemm_dense_conv_i8" in families(k), k


@pytest.mark.parametrize("variant", [4, 5, 6, 7, 8, 9, 10])
def test_conv2d_window_ring_every_tile(device, variant, monkeypatch):
    monkeypatch.setenv("THIP_WINDOW_VARIANT", str(variant))
    names = {4: "igemm_dense_conv_i8<256,256,", 5: "igemm_dense_conv_i8<128,128,", 6: "igemm_dense_conv_i8<128,256,", 7: "igemm_dense_conv_i8<64,64,",
             8: "igemm_dense_conv_i8<256,128,", 9: "igemm_dense_conv_i8<256,64,", 10: "igemm_dense_conv_i8<256,32,"}
    for kw in (dict(N=2, H=33, W=35, C=64, O=80, pad=(1, 1, 1, 1)), dict(N=5, H=47, W=45, C=128, O=48, stride=(2, 2), pad=(1, 0, 1, 0), output_zp=-7, output_min=-128),
               dict(N=3, H=29, W=31, C=80, O=72, pad=(1, 1, 1, 1), input_zp=-90), dict(N=4, H=40, W=33, C=176, O=130, KH=2, KW=2, stride=(1, 2), pad=(0, 1, 1, 0))):
        k = check(device, w.conv2d_workload(realistic=True, **kw), via="device")
        assert k[0].startswith(names[variant]), k
    # an int32 result and a requant shift on the 64-bit tail: the staged epilogue
    k = check(device, w.conv2d_workload(N=2, H=32, W=32, C=64, O=64, realistic=False))
    assert k[0].startswith(names[variant]), k


def test_conv2d_window_ring_k128(device, monkeypatch):
    """C % 128 == 0 and at least 128 tiles of 256 x 256: k-tiles of 128 channels of one tap (asked for by hand, of any
    128 channels or more)."""
    k = check(device, w.conv2d_workload(N=8, H=64, W=64, C=128, O=256, realistic=True), via="device")
    assert k[0] == "igemm_dense_conv_i8<256,256,2,2,2,1,1,0>", k
    monkeypatch.setenv("THIP_WINDOW_VARIANT", "14")
    for kw in (dict(N=2, H=33, W=35, C=128, O=80, pad=(1, 1, 1, 1)), dict(N=5, H=47, W=45, C=256, O=48, stride=(2, 2), pad=(1, 0, 1, 0), output_zp=-7, output_min=-128),
               dict(N=3, H=30, W=30, C=384, O=40, KH=2, KW=5, pad=(3, 1, 0, 1)), dict(N=2, H=34, W=31, C=144, O=96, pad=(1, 1, 1, 1), input_zp=101),
               dict(N=4, H=31, W=35, C=208, O=300, KH=1, KW=3, stride=(2, 1), pad=(1, 0, 0, 0))):
        k = check(device, w.conv2d_workload(realistic=True, **kw), via="device")
        assert k[0].startswith("igemm_dense_conv_i8<256,256,2,2,2,1,"), k
    k = check(device, w.conv2d_workload(N=2, H=32, W=32, C=128, O=64, realistic=False))  # the literal requant range
    assert k[0].startswith("igemm_dense_conv_i8<256,256,2,2,2,1,"), k
    k = check(device, w.conv2d_workload(N=2, H=32, W=32, C=64, O=64, realistic=True))    # half a k-tile per tap
    assert k[0].startswith("igemm_dense_conv_i8<256,256,2,2,2,1,"), k
    monkeypatch.delenv("THIP_WINDOW_VARIANT")
    k = check(device, w.conv2d_workload(N=2, H=32, W=32, C=64, O=64, realistic=True))
    assert k[0].startswith("igemm_dense_conv_i8<64,64,2,2,4,4,"), k   # 32 small tiles
    k = check(device, w.conv2d_workload(N=20, H=32, W=32, C=64, O=128, realistic=True))
    assert k[0].startswith("igemm_dense_conv_i8<128,128,"), k         # 640 small tiles would be too many, 160 of 128 x 128
    k = check(device, w.conv2d_workload(N=30, H=48, W=48, C=64, O=64, realistic=True), via="device")  # 270 row tiles: one tile column
    assert k[0].startswith("igemm_dense_conv_i8<256,64,"), k
    k = check(device, w.conv2d_workload(N=1, H=14, W=14, C=256, O=256, realistic=True))  # few pixels, a long K: the small tile
    assert k[0].startswith("igemm_dense_conv_i8<64,64,2,2,4,4,"), k
    k = check(device, w.conv2d_workload(N=1, H=14, W=14, C=256, O=250, realistic=False))  # the small tile's staged epilogue
    assert k[0].startswith("igemm_dense_conv_i8<64,64,2,2,4,4,0,"), k


@pytest.mark.parametrize("variant,name", [(5, "igemm_dense_conv_i8<128,128,2,2,2,2,"), (6, "igemm_dense_conv_i8<128,256,2,2,2,1,")])
def test_conv2d_window_ring_128_wide_tiles_long_k(device, variant, name, monkeypatch):
    """The 128-wide window tiles with K >= 2304 in whole 128-byte k-tiles: 128 channels of the window per k-tile row."""
    monkeypatch.setenv("THIP_WINDOW_VARIANT", str(variant))
    for kw in (dict(N=3, H=29, W=31, C=256, O=144, pad=(1, 1, 1, 1), input_zp=-90), dict(N=5, H=27, W=25, C=128, O=48, KH=5, KW=4, stride=(2, 2), pad=(1, 0, 2, 0), output_zp=-7, output_min=-128),
               dict(N=2, H=20, W=33, C=384, O=130, KH=3, KW=3, stride=(1, 2), pad=(0, 1, 1, 0)), dict(N=2, H=30, W=30, C=96, O=64, KH=4, KW=7, pad=(3, 3, 1, 2))):
        k = check(device, w.conv2d_workload(realistic=True, **kw), via="device")
        assert k[0].startswith(name), (kw, k)
    k = check(device, w.conv2d_workload(N=2, H=32, W=32, C=256, O=64, realistic=False))   # the literal requant range
    assert k[0].startswith(name), k
    k = check(device, w.conv2d_workload(N=2, H=32, W=32, C=208, O=64, realistic=True))    # K = 1872: 64-byte k-tiles
    assert not k[0].startswith(name), k


@pytest.mark.parametrize("variant", [None, 14, 9])
def test_conv2d_window_ring_few_channels(device, variant, monkeypatch):
    """Fewer channels than a k-tile: the chunks of one k-tile span several taps and window rows."""
    if variant is not None:
        monkeypatch.setenv("THIP_WINDOW_VARIANT", str(variant))
    for kw in WINDOW_RING_FEW_CHANNELS:
        k = check(device, w.conv2d_workload(realistic=True, **kw), via="device")
        assert families(k) == ["igemm_dense_conv_i8"], (kw, k)


def test_conv2d_window_ring_switch(device, monkeypatch):
    monkeypatch.setenv("THIP_NO_WINDOW_RING", "1")
    k = check(device, w.conv2d_workload(N=2, H=32, W=32, C=64, O=64, realistic=True))
    assert families(k) == ["igemm_i8"], k


@pytest.mark.parametrize("variant", [4, 5, 6, 7, 8, 9, 10, 12, 13])
def test_dense_igemm_every_tile_variant(device, variant, monkeypatch):
    """The LDS-DMA kernel: whole tiles, ragged M / N / K tails, K shorter than the stage ring."""
    monkeypatch.setenv("THIP_IGEMM_DENSE_VARIANT", str(variant))
    tile = {4: (256, 256), 5: (128, 128), 6: (128, 256), 7: (64, 64), 8: (256, 128), 9: (256, 64), 10: (256, 32), 12: (128, 64), 13: (64, 128)}[variant]
    k = check(device, w.fully_connected_workload(300, 192, 520, realistic=True))
    assert k[0].startswith("igemm_dense_i8<%d,%d," % tile) and k[0].endswith(",0,0>"), k  # N % 16 != 0: results leave through LDS
    k = check(device, w.fully_connected_workload(512, 1024, 512, realistic=True))
    assert k[0].startswith("igemm_dense_i8<%d,%d," % tile) and k[0].endswith(",1,0>"), k  # N % 16 == 0, shift >= 33: the in-register epilogue
    k = check(device, w.fully_connected_workload(300, 320, 528))
    assert k[0].startswith("igemm_dense_i8<%d,%d," % tile) and k[0].endswith(",2,0>"), k  # the literal requant range: the general 32-bit tail, in registers
    for shift in (32, 40, 50, 62):
        k = check(device, w.fully_connected_workload(130, 96, 64, shift=shift, output_zp=-7))
        assert k[0].endswith(",2,0>" if shift > 45 or shift == 32 else ",1,0>"), (shift, k)
    check(device, w.fully_connected_workload(257, 80, 48, realistic=True))
    check(device, w.fully_connected_workload(33, 16, 1000, realistic=True))
    check(device, w.fully_connected_workload(1000, 4096, 272, realistic=True))
    check(device, w.conv2d_workload(N=2, H=28, W=28, C=192, O=32, KH=1, KW=1, pad=(0, 0, 0, 0), realistic=True))


def test_dense_igemm_64x128_long_k(device, monkeypatch):
    """The 64 x 128 tile with a long K in whole 128-byte k-tiles: ragged M and N, every epilogue; other K keep 64 bytes."""
    k = check(device, w.fully_connected_workload(512, 4096, 4096, realistic=True), via="device")
    assert k[0] == "igemm_dense_k128_i8<64,128,2,2,3,2,1,0>", k                          # chosen without a switch
    monkeypatch.setenv("THIP_IGEMM_DENSE_VARIANT", "13")
    k = check(device, w.fully_connected_workload(500, 4096, 2064, realistic=True), via="device")
    assert k[0] == "igemm_dense_k128_i8<64,128,2,2,3,2,1,0>", k
    k = check(device, w.fully_connected_workload(500, 4224, 2064))                       # the literal requant range
    assert k[0] == "igemm_dense_k128_i8<64,128,2,2,3,2,2,0>", k
    k = check(device, w.fully_connected_workload(300, 4096, 2056, realistic=True))       # N % 16 != 0: staged epilogue
    assert k[0] == "igemm_dense_k128_i8<64,128,2,2,3,2,0,0>", k
    k = check(device, w.fully_connected_workload(500, 4160, 2064, realistic=True))       # K % 128 != 0
    assert k[0] == "igemm_dense_i8<64,128,2,2,4,2,1,0>", k
    monkeypatch.setenv("THIP_NO_K128", "1")
    k = check(device, w.fully_connected_workload(500, 4096, 2064, realistic=True))
    assert k[0] == "igemm_dense_i8<64,128,2,2,4,2,1,0>", k


def test_dense_igemm_128_wide_tiles_long_k(device, monkeypatch):
    """The 128 x 128 and 128 x 256 tiles with a long K in whole 128-byte k-tiles: ragged M and N, every epilogue."""
    k = check(device, w.fully_connected_workload(1500, 4096, 4096, realistic=True), via="device")
    assert k[0] == "igemm_dense_k128_i8<128,128,2,2,2,2,1,0>", k                         # chosen without a switch
    k = check(device, w.fully_connected_workload(1000, 4096, 4096, realistic=True), via="device")
    assert k[0] == "igemm_dense_i8<128,128,2,2,4,2,1,0>", k                              # one tile per CU: the deeper ring
    monkeypatch.setenv("THIP_IGEMM_DENSE_VARIANT", "5")
    k = check(device, w.fully_connected_workload(1100, 4224, 4112))                      # the literal requant range
    assert k[0] == "igemm_dense_k128_i8<128,128,2,2,2,2,2,0>", k
    k = check(device, w.fully_connected_workload(1100, 4096, 4104, realistic=True))      # N % 16 != 0: staged epilogue
    assert k[0] == "igemm_dense_k128_i8<128,128,2,2,2,2,0,0>", k
    monkeypatch.setenv("THIP_IGEMM_DENSE_VARIANT", "6")
    for wl, tail in ((w.fully_connected_workload(700, 4096, 2064, realistic=True), "1,0>"), (w.fully_connected_workload(700, 4224, 2064), "2,0>"),
                     (w.fully_connected_workload(300, 4096, 2056, realistic=True), "0,0>")):
        k = check(device, wl)
        assert k[0] == "igemm_dense_k128_i8<128,256,2,2,2,1," + tail, k
    k = check(device, w.fully_connected_workload(700, 4160, 2064, realistic=True))       # K % 128 != 0
    assert k[0] == "igemm_dense_i8<128,256,2,2,3,2,1,0>", k


def test_dense_igemm_short_k(device, monkeypatch):
    """Up to six k-tiles over at least two 128 x 128 tiles per CU: two ring stages, four blocks per CU (K of one to six
    k-tiles, ragged M / N / K, every epilogue); fewer tiles or a longer K keep the deeper ring."""
    for K in (16, 64, 100 // 4 * 4 + 12, 192, 256, 320, 384):
        k = check(device, w.fully_connected_workload(16500, K, 512, realistic=True), via="device")
        assert k[0] == "igemm_dense_i8<128,128,2,2,2,4,1,0>", (K, k)
    k = check(device, w.fully_connected_workload(16500, 256, 512))                      # the literal requant range
    assert k[0] == "igemm_dense_i8<128,128,2,2,2,4,2,0>", k
    monkeypatch.setenv("THIP_IGEMM_DENSE_VARIANT", "5")
    k = check(device, w.fully_connected_workload(16390, 208, 520, realistic=True))      # N % 16 != 0: staged epilogue
    assert k[0] == "igemm_dense_i8<128,128,2,2,2,4,0,0>", k
    k = check(device, w.fully_connected_workload(16390, 448, 512, realistic=True))      # seven k-tiles
    assert k[0] == "igemm_dense_i8<128,128,2,2,4,2,1,0>", k
    k = check(device, w.fully_connected_workload(8000, 256, 512, realistic=True))       # 252 tiles
    assert k[0] == "igemm_dense_i8<128,128,2,2,4,2,1,0>", k
    monkeypatch.setenv("THIP_DENSE_SHORT_K", "0")
    k = check(device, w.fully_connected_workload(16500, 256, 512, realistic=True))
    assert k[0] == "igemm_dense_i8<128,128,2,2,4,2,1,0>", k


def test_dense_igemm_k128(device, monkeypatch):
    """k-tiles of 128 bytes (whole cache lines per tile row, four MFMA phases, two ring stages): taken by itself for a
    long K with enough tiles, forced here on ragged M / N, K tails that end inside a k-tile (at every 16-byte chunk),
    K shorter than one k-tile and than the ring, every epilogue."""
    k = check(device, w.fully_connected_workload(4096, 1024, 4096, realistic=True), via="device")
    assert k[0] == "igemm_dense_k128_i8<256,256,2,2,2,1,1,0>", k       # chosen without a switch
    k = check(device, w.fully_connected_workload(4096, 1024, 4096), via="device")
    assert k[0] == "igemm_dense_k128_i8<256,256,2,2,2,1,2,0>", k       # the literal requant range: the general 32-bit tail
    monkeypatch.setenv("THIP_IGEMM_DENSE_VARIANT", "14")
    for K in (16, 48, 112, 128, 144, 240, 256, 272, 400, 1024 + 64, 2048 + 16):
        k = check(device, w.fully_connected_workload(300, K, 272, realistic=True))
        assert k[0].startswith("igemm_dense_k128_i8<256,256,2,2,2,1,"), k
    k = check(device, w.fully_connected_workload(300, 192, 520, realistic=True))
    assert k[0].endswith(",0,0>"), k                                    # N % 16 != 0: the staged epilogue
    check(device, w.fully_connected_workload(513, 1024, 515, realistic=True))
    check(device, w.fully_connected_workload(17, 4096, 16, realistic=True))
    check(device, w.conv2d_workload(N=2, H=28, W=28, C=192, O=32, KH=1, KW=1, pad=(0, 0, 0, 0), realistic=True))
    check(device, w.matmul_workload(2, 70, 200, 90))                    # run-time input2: transposed into rows of Kp = 256
    monkeypatch.setenv("THIP_NO_K128", "1")
    monkeypatch.delenv("THIP_IGEMM_DENSE_VARIANT")
    k = check(device, w.fully_connected_workload(4096, 1024, 4096, realistic=True), via="device")
    assert k[0] == "igemm_dense_i8<256,256,2,2,4,1,1,0>", k


@pytest.mark.parametrize("variant", [4, 7, 9, 13])
def test_dense_igemm_staged_epilogue(device, variant, monkeypatch):
    """The LDS-staged epilogue with the 32-bit requant tail (the in-register one normally takes these shapes)."""
    monkeypatch.setenv("THIP_IGEMM_DENSE_VARIANT", str(variant))
    monkeypatch.setenv("THIP_NO_DIRECT_EPILOGUE", "1")
    for mkn in [(300, 192, 528), (257, 80, 48)]:
        k = check(device, w.fully_connected_workload(*mkn, realistic=True), kernel="igemm_dense_i8")
        assert k[0].endswith(",0,0>"), k  # the staged epilogue


@pytest.mark.parametrize("guarded", [False, True, "staged"])
def test_stream_igemm(device, guarded, monkeypatch):
    """The pixel-streaming kernel (weights resident in LDS): every accumulator width, ragged M (also fewer rows than
    one group), k-step counts around the prefetch ring (one and two k-steps take a ring over several groups), N
    ending in half a 32-channel block, both requant tails; with the branch-free steady state and with every load
    and store under its bounds check, and with the results leaving through the per-wave LDS slices wherever these fit."""
    monkeypatch.setenv("THIP_IGEMM_DENSE_VARIANT", "11")
    if guarded == "staged":
        monkeypatch.setenv("THIP_STREAM_STAGE", "1")
    elif guarded:
        monkeypatch.setenv("THIP_STREAM_GUARDED", "1")
    for M, K, N in [(17, 16, 16), (31, 64, 80), (32, 32, 96), (65, 48, 32), (4096 + 5, 64, 224)]:
        check(device, w.fully_connected_workload(M, K, N, realistic=True), kernel="igemm_stream_i8")
    for M, K, N in [(33, 16, 16), (257, 80, 48), (1000, 144, 32), (4099, 96, 112), (5000, 32, 144),
                    (300, 192, 240), (2048, 224, 256), (70000, 32, 16),
                    (900, 64, 384), (700, 96, 592), (513, 32, 1008)]:
        check(device, w.fully_connected_workload(M, K, N, realistic=True), kernel="igemm_stream_i8")
    for shift in [0, 1, 31, 32, 33, 34, 62]:
        check(device, w.fully_connected_workload(500, 48, 80, shift=shift, output_zp=-7), kernel="igemm_stream_i8")
    # chosen without forcing for an expanding pointwise convolution from 40 000 pixels, for one with at most four k-steps
    # from 200 000; not below that, not for a projecting one with a long K, and not when the weights outgrow LDS
    monkeypatch.delenv("THIP_IGEMM_DENSE_VARIANT")
    check(device, w.conv2d_workload(N=13, H=56, W=56, C=32, O=144, KH=1, KW=1, pad=(0, 0, 0, 0), realistic=True), kernel="igemm_stream_i8")
    check(device, w.conv2d_workload(N=4, H=56, W=56, C=32, O=144, KH=1, KW=1, pad=(0, 0, 0, 0), realistic=True), kernel="igemm_dense_i8")
    check(device, w.conv2d_workload(N=13, H=56, W=56, C=96, O=32, KH=1, KW=1, pad=(0, 0, 0, 0), realistic=True), kernel="igemm_dense_i8")
    check(device, w.conv2d_workload(N=70, H=56, W=56, C=96, O=32, KH=1, KW=1, pad=(0, 0, 0, 0), realistic=True), kernel="igemm_stream_i8")
    check(device, w.conv2d_workload(N=70, H=56, W=56, C=144, O=32, KH=1, KW=1, pad=(0, 0, 0, 0), realistic=True), kernel="igemm_dense_i8")
    check(device, w.fully_connected_workload(8192, 256, 256, realistic=True), kernel="igemm_dense_i8")
    # few input channels: the streaming kernel gathers one run per window row (also across the image border)
    for kw in [dict(N=2, H=224, W=224, C=3, O=32, stride=(2, 2), pad=(0, 1, 0, 1), input_zp=-1),
               dict(N=1, H=70, W=70, C=4, O=48, KH=5, KW=3, stride=(1, 1), pad=(1, 1, 2, 2), input_zp=9),
               dict(N=3, H=80, W=81, C=2, O=16, KH=7, KW=7, stride=(2, 2), pad=(3, 3, 3, 3), input_zp=-128),
               dict(N=1, H=75, W=66, C=1, O=64, KH=3, KW=3, stride=(1, 1), pad=(0, 0, 0, 0))]:
        check(device, w.conv2d_workload(realistic=True, **kw), kernel="igemm_stream_i8")
    monkeypatch.setenv("THIP_NO_STREAM", "1")
    check(device, w.conv2d_workload(N=2, H=224, W=224, C=3, O=32, stride=(2, 2), pad=(0, 1, 0, 1), realistic=True, input_zp=-1), kernel="igemm_i8")


@pytest.mark.parametrize("shift", [0, 1, 6, 31, 32, 33, 34, 40, 62])
def test_igemm_shift_boundaries(device, shift):
    """Both epilogue tails of the MFMA kernels (generic 64-bit, and 32-bit for shift >= 33) around their switch."""
    check(device, w.fully_connected_workload(200, 256, 144, shift=shift), kernel="igemm_dense_i8")
    check(device, w.fully_connected_workload(40, 72, 20, shift=shift, output_zp=-7), kernel="igemm_i8")
    check(device, w.fully_connected_workload(3, 64, 40, shift=shift), kernel="fc_skinny_mfma")


def test_conv2d_mbv2_layer_shapes(device):
    # first layer (3 channels, stride 2, TF SAME), expand / project 1x1, last 1x1
    check(device, w.conv2d_workload(N=2, H=224, W=224, C=3, O=32, stride=(2, 2), pad=(0, 1, 0, 1), realistic=True, input_zp=-1))
    check(device, w.conv2d_workload(N=2, H=56, W=56, C=24, O=144, KH=1, KW=1, pad=(0, 0, 0, 0), realistic=True))
    check(device, w.conv2d_workload(N=2, H=28, W=28, C=192, O=32, KH=1, KW=1, pad=(0, 0, 0, 0), realistic=True))
    check(device, w.conv2d_workload(N=2, H=7, W=7, C=320, O=1280, KH=1, KW=1, pad=(0, 0, 0, 0), realistic=True))


def test_conv2d_on_images_smaller_than_one_load(device):
    for kw in (dict(N=1, H=2, W=6, C=1, O=3, KH=2, KW=1, pad=(0, 0, 1, 0)), dict(N=1, H=11, W=1, C=1, O=15, KH=3, KW=1, pad=(0, 0, 1, 1)),
               dict(N=2, H=1, W=1, C=4, O=3, KH=1, KW=1, pad=(0, 0, 0, 0)), dict(N=1, H=2, W=2, C=3, O=24, KH=2, KW=1, pad=(0, 0, 0, 1)),
               dict(N=1, H=4, W=4, C=1, O=5, KH=3, KW=3), dict(N=1, H=1, W=1, C=1, O=1, KH=1, KW=1, pad=(0, 0, 0, 0))):
        check(device, w.conv2d_workload(realistic=True, **kw), kernel="igemm_i8")


def test_conv2d_int32_output(device):
    wl = w.conv2d_workload(N=1, H=9, W=9, C=16, O=8, realistic=True)
    # same op, int32 init and full-range clamp: exposes the un-narrowed requant result
    from torq_compiler_amd import Program
    a = dict(wl.attrs)
    wts, sb = a.pop("weights"), a.pop("scale_bias")
    a.pop("nhwc")
    a.update(output_min=-(1 << 31), output_max=(1 << 31) - 1)
    a["shift_factor"] = max(a["shift_factor"] - 8, 0)
    p = Program()
    out = p.binding(1, (1, 9, 9, 8), np.int32)
    p.conv2d(p.binding(0, (1, 9, 9, 16)), wts, sb, init=out, nhwc_input=True, out_dtype=np.int32, **a)
    from oracle import oracle as orc
    want = orc.conv2d(wl.inputs[0], wts, sb, layout=orc.NHWC, out_dtype=np.int32, **a)
    announce("conv2d int32 out")
    exe = Executable(device, p.serialize())
    got = np.zeros((1, 9, 9, 8), dtype=np.int32)
    exe.run_host([wl.inputs[0], got])
    exe.close()
    assert_bit_exact(got, want, "conv2d int32")


# ---- fully_connected ---------------------------------------------------------------------------
@pytest.mark.parametrize("mkn", [(1, 2048, 2048), (16, 2048, 8192), (512, 4096, 4096)])
def test_fully_connected_config1(device, mkn):
    M = mkn[0]
    check(device, w.fully_connected_workload(*mkn, realistic=True), via="device",
          kernel=("fc_skinny<1,4>" if M == 1 else "fc_skinny_mfma") if M <= 16 else ("igemm_dense_k128_i8" if M >= 512 else None))


@pytest.mark.parametrize("mkn", [(1, 2048, 2048), (16, 2048, 8192), (512, 4096, 4096)])
def test_fully_connected_config1_literal_ranges(device, mkn):
    # the benchmark's own requant range (shift 6 .. 12 under multipliers of 2^30 and more): every output saturates, and the
    # dense tiles requantise it through the pre-shifted 32-bit tail with the accumulator clamped first
    check(device, w.fully_connected_workload(*mkn), via="device")


@pytest.mark.parametrize("mkn", [(1, 1, 1), (1, 61, 1991), (4, 1024, 1024), (1, 2000, 97), (16, 3, 7), (17, 128, 70),
                                 (130, 700, 500), (3, 1280, 1000), (9, 1000, 512)])
def test_fully_connected_geometries(device, mkn):
    check(device, w.fully_connected_workload(*mkn, realistic=True))


@pytest.mark.parametrize("dot4", [False, True])
def test_fully_connected_skinny_kernels(device, dot4, monkeypatch):
    """At most 16 rows: the MFMA kernel (2 rows and up) and the dot-product kernel, K and N with ragged ends."""
    if dot4:
        monkeypatch.setenv("THIP_SKINNY_DOT4", "1")
    def expected(M):
        if M >= 2 and not dot4:
            return "fc_skinny_mfma"
        return "fc_skinny<1,4>" if M == 1 else "fc_skinny<4,4>" if M <= 4 else "fc_skinny<8,2>" if M <= 8 else "fc_skinny<16,2>"
    for mkn in [(3, 16, 16), (5, 48, 20), (16, 272, 1000), (9, 1040, 37), (4, 256, 64), (2, 512, 32), (16, 2048, 8192), (7, 4096, 130), (1, 64, 48)]:
        check(device, w.fully_connected_workload(*mkn, realistic=True), kernel=expected(mkn[0]))
    check(device, w.fully_connected_workload(12, 528, 100, shift=7), kernel=expected(12))


def test_fully_connected_without_skinny_kernel(device, monkeypatch):
    monkeypatch.setenv("THIP_NO_SKINNY", "1")
    check(device, w.fully_connected_workload(16, 2048, 512, realistic=True), kernel="igemm_dense_i8")


# ---- matmul (int8) ----------------------------------------------------------------------------
@pytest.mark.parametrize("kw", MATMUL, ids=matmul_id)
def test_matmul_int8(device, kw):
    """torq_hl.matmul with ONE (bias, scale) pair (compiler/torq/Conversions/TorqHLToTorqHW/MatMulPattern.cpp:66-86): the
    reference's fixture shapes, batch broadcast on either side, constant and run-time input2, every result type."""
    wl = w.matmul_workload(**kw)
    kernels = check(device, wl, via="device" if kw["M"] >= 64 else "host")
    if not kw.get("constant_rhs"):
        assert kernels[0] == "transpose_i8<1>"
    assert any(k.startswith("igemm") for k in kernels)


# ---- bandwidth ops ---------------------------------------------------------------------------
@pytest.mark.parametrize("batch", [1, 8, 64])
def test_depthwise_config2a(device, batch):
    """56x56x144 stride 2 at the benchmark's batch sizes; batch 64 has enough waves for the rolling-window kernel."""
    check(device, w.depthwise_workload(N=batch), via="device",
          kernel="depthwise3x3_strip_i8<2,2,1,3,1>" if batch == 64 else "depthwise3x3_dot4_i8<1,0>")


@pytest.mark.parametrize("kw", [
    dict(N=1, H=6, W=42, C=16), dict(N=1, H=6, W=6, C=2, pad=(0, 0, 0, 0)), dict(N=1, H=13, W=15, C=8, stride=(1, 1), pad=(1, 1, 1, 1)),
    dict(N=1, H=27, W=27, C=128, KH=4, KW=4, stride=(2, 2), pad=(1, 2, 1, 2)), dict(N=2, H=21, W=21, C=5, stride=(2, 2), pad=(1, 1, 1, 1)),
    dict(N=1, H=14, W=14, C=36, stride=(1, 1), pad=(1, 1, 1, 1)), dict(N=3, H=112, W=112, C=32, stride=(1, 1), pad=(1, 1, 1, 1)),
])
@pytest.mark.parametrize("nhwc", [True, False])
def test_depthwise_geometries(device, kw, nhwc):
    check(device, w.depthwise_workload(nhwc=nhwc, **kw))


@pytest.mark.parametrize("which", ["rows", "tile", "strip", "strip1"])
def test_depthwise_3x3_kernels(device, which, monkeypatch):
    """The three 3x3 kernels (one window row of pixels per thread, a register tile of outputs per thread, a rolling
    window down a segment of rows, with two columns or, at stride 2, one column per thread) on images whose sizes
    are no multiples of the tiles or segments, with and without padding, stride 1 and 2, with one and with several
    row segments."""
    monkeypatch.setenv("THIP_DEPTHWISE_TILE", "1" if which == "tile" else "0")
    monkeypatch.setenv("THIP_DEPTHWISE_STRIP", {"strip": "1", "strip1": "2"}.get(which, "0"))
    seen = set()
    for kw in [dict(N=2, H=13, W=15, C=16, stride=(1, 1), pad=(1, 1, 1, 1)), dict(N=1, H=14, W=14, C=48, stride=(1, 1), pad=(0, 0, 0, 0)),
               dict(N=1, H=9, W=31, C=32, stride=(1, 1), pad=(1, 1, 1, 1)), dict(N=2, H=21, W=22, C=16, stride=(2, 2), pad=(0, 1, 0, 1)),
               dict(N=1, H=15, W=13, C=80, stride=(2, 2), pad=(1, 1, 1, 1)), dict(N=1, H=3, W=3, C=16, stride=(1, 1), pad=(0, 0, 0, 0)),
               dict(N=1, H=56, W=56, C=144, stride=(1, 1), pad=(1, 1, 1, 1), realistic=False),
               dict(N=1, H=8, W=8, C=16, stride=(2, 2), pad=(1, 1, 1, 1), input_zp=-128),
               dict(N=3, H=30, W=17, C=96, stride=(1, 1), pad=(1, 1, 1, 1), input_zp=7),
               dict(N=2, H=41, W=9, C=16, stride=(1, 1), pad=(1, 1, 1, 1), input_zp=-5),
               dict(N=1, H=45, W=7, C=32, stride=(2, 2), pad=(1, 1, 1, 1), input_zp=3),
               dict(N=1, H=1, W=5, C=16, stride=(1, 1), pad=(1, 1, 1, 1)),
               dict(N=2, H=112, W=112, C=32, stride=(2, 2), pad=(0, 1, 0, 1), input_zp=-128)]:
        seen.add(check(device, w.depthwise_workload(**kw), kernel=depthwise_kernel(which, kw["stride"][0]))[0])
    assert len(seen) >= (1 if which == "rows" else 2), seen  # both strides took a kernel of their own


def depthwise_kernel(which, stride):
    """The 3x3 depthwise kernel the switches of test_depthwise_3x3_kernels select at this stride."""
    if which == "tile":
        return "depthwise3x3_tile_i8<4,2,1,4>" if stride == 1 else "depthwise3x3_dot4_i8"
    if which == "strip":
        return "depthwise3x3_strip_i8<2,1,1,4,3>" if stride == 1 else "depthwise3x3_strip_i8<2,2,1,3,1>"
    if which == "strip1":
        return "depthwise3x3_strip_i8<2,1,1,4,3>" if stride == 1 else "depthwise3x3_strip_i8<1,2,1,4,3>"
    return "depthwise3x3_dot4_i8"


@pytest.mark.parametrize("which", ["rows", "tile", "strip", "strip1"])
def test_depthwise_shift_boundaries(device, which, monkeypatch):
    """Every requant tail of the 3x3 kernels: the generic 64-bit one, the bits of the sum read directly (a shift below
    32 with a proven bound), with a clamp of acc + bias (a large bias breaks the bound), the high word itself
    (shift 32) and the shifted high word (33 and up); zero points of either sign."""
    monkeypatch.setenv("THIP_DEPTHWISE_TILE", "1" if which == "tile" else "0")
    monkeypatch.setenv("THIP_DEPTHWISE_STRIP", {"strip": "1", "strip1": "2"}.get(which, "0"))
    stride = (2, 2) if which == "strip1" else (1, 1)
    for shift in [0, 2, 3, 12, 24, 31, 32, 33, 34, 40, 62]:
        for zp in (-7, 100):
            check(device, w.depthwise_workload(N=1, H=12, W=10, C=32, stride=stride, pad=(1, 1, 1, 1), shift=shift, output_zp=zp),
                  kernel=depthwise_kernel(which, stride[0]))
    check(device, w.depthwise_workload(N=1, H=12, W=10, C=32, stride=(2, 2), pad=(1, 1, 1, 1), shift=31, output_zp=-128),
          kernel=depthwise_kernel(which, 2))
    monkeypatch.setenv("THIP_NO_PRE_SHIFT", "1")
    check(device, w.depthwise_workload(N=1, H=12, W=10, C=32, stride=(1, 1), pad=(1, 1, 1, 1), shift=24), kernel=depthwise_kernel(which, 1))


@pytest.mark.parametrize("batch", [1, 8, 64])
def test_maxpool_config2b(device, batch, monkeypatch):
    """112x112x64, 2x2 stride 2, at the benchmark's batch sizes: the dedicated 2x2 kernel, and the any-window one."""
    check(device, w.maxpool_workload(N=batch), via="device", kernel="maxpool2x2_i8")
    if batch == 8:
        monkeypatch.setenv("THIP_MAXPOOL_GENERIC", "1")
        check(device, w.maxpool_workload(N=batch), via="device", kernel="maxpool_i8<16>")


def test_maxpool_2x2_kernel_edges(device):
    """The 2x2 kernel's packed byte maxima on the extremes (-128 and 127 next to each other in every byte position),
    odd image sizes (the last row / column is never read), and the shapes it must leave to the general kernel."""
    wl = w.maxpool_workload(N=2, H=9, W=11, C=32)
    x = wl.inputs[0]
    x[...] = np.array([-128, 127, -1, 0, 1, -127, 126, -2], dtype=np.int8)[np.arange(x.size).reshape(x.shape) % 8]
    x[0, ::2, ::2, ::3] = -128
    x[1, 1::2, :, 1::2] = 127
    check(device, wl, kernel="maxpool2x2_i8")
    check(device, w.maxpool_workload(N=1, H=16, W=16, C=16), kernel="maxpool2x2_i8")
    check(device, w.maxpool_workload(N=1, H=16, W=16, C=16, pad=(0, 1, 0, 1)), kernel="maxpool2x2_i8")    # declared, never reached
    check(device, w.maxpool_workload(N=1, H=15, W=15, C=16, pad=(0, 1, 0, 1)), kernel="maxpool_i8<16>")   # padding is touched
    check(device, w.maxpool_workload(N=1, H=16, W=16, C=24), kernel="maxpool_i8<8>")                       # C % 16 != 0
    check(device, w.maxpool_workload(N=1, H=16, W=16, C=16, kernel=(3, 3), stride=(2, 2)), kernel="maxpool_i8<16>")


@pytest.mark.parametrize("kw", [dict(H=8, W=8, C=4), dict(H=8, W=8, C=1), dict(H=32, W=32, C=64, kernel=(3, 3), pad=(1, 1, 1, 1)),
                                dict(H=10, W=10, C=4, kernel=(5, 5), stride=(1, 1)), dict(H=224, W=224, C=64, kernel=(3, 3), pad=(0, 1, 0, 1)),
                                dict(H=10, W=10, C=4, kernel=(1, 3), stride=(1, 3), pad=(0, 2, 0, 0), input_zp=-7)])
@pytest.mark.parametrize("nhwc", [True, False])
def test_maxpool_geometries(device, kw, nhwc):
    check(device, w.maxpool_workload(nhwc=nhwc, **kw))


@pytest.mark.parametrize("kw", [dict(N=1), dict(N=64), dict(N=2, C=128), dict(N=1, H=12, W=8, C=37), dict(N=3, H=37, W=17, C=11), dict(N=1, H=53, W=37, C=1)])
def test_avgpool(device, kw):
    check(device, w.avgpool_workload(**kw), kernel="avgpool_i8")


@pytest.mark.parametrize("kw", [dict(N=1), dict(N=64), dict(N=1, H=4, W=4, C=1), dict(N=1, H=6, W=8, C=4, zp0=127, zp1=-128), dict(N=1, H=7, W=7, C=33)])
def test_add(device, kw, monkeypatch):
    """The quantised add with the patterns' scale 1 / shift 12 (one folded 32-bit constant), and through the 64-bit ACT stage."""
    check(device, w.add_workload(**kw), via="device", kernel="add_i8<16,1>")
    monkeypatch.setenv("THIP_ADD_GENERIC", "1")
    check(device, w.add_workload(**kw), via="device", kernel="add_i8<16,0>")


# ---- programs, properties, error paths ------------------------------------------------------------
def test_multi_op_program(device):
    p, x, want_fc, want_sum = _chain_program(True)
    announce("inverted-residual chain program")
    exe = Executable(device, p.serialize())
    out = np.zeros(want_fc.shape, dtype=np.int8)
    aux = np.zeros(want_sum.shape, dtype=np.int8)
    exe.run_host([x, out, aux])
    assert_bit_exact(out, want_fc, "chain fc")
    assert_bit_exact(aux, want_sum, "chain residual")
    # running again gives the same bytes (intermediates hold no state between dispatches)
    out2 = np.zeros_like(out)
    exe.run_host([x, out2, np.zeros_like(aux)])
    exe.close()
    assert np.array_equal(out, out2)


@pytest.mark.parametrize("nhwc", [True, False])
def test_padded_channel_chain(device, nhwc):
    """24-channel intermediates stored as 32: depthwise, max pool, 3x3 conv, add and pointwise conv on them."""
    p, x, want = _padded_chain(nhwc)
    announce("padded-channel chain nhwc=%s" % nhwc)
    exe = Executable(device, p.serialize())
    out = np.zeros(want.shape, dtype=np.int8)
    exe.run_host([x, out])
    exe.close()
    assert_bit_exact(out, want, "padded chain")


@pytest.mark.parametrize("batch", [1, 3, 32])
def test_mobilenet_v2_full(device, batch):
    """benchmark configuration 3: the whole 64-op network as one program, final logits of every image bit-exact."""
    wl = w.mobilenet_v2_workload(batch=batch)
    announce(wl.name)
    got, kernels = run_on_gpu(device, wl, via="device")
    assert_bit_exact(got[0], oracle_network(wl), wl.name)
    # 64 ops; a residual add behind a streaming convolution (enough pixels) is folded into it
    assert 54 <= len(kernels) <= 64 and "transpose_i8" not in families(kernels)


def test_mobilenet_v2_batch256(device):
    """benchmark configuration 3 at its largest batch: the first and the last four images against the oracle, and every
    image independent of its neighbours (copies of an image at other batch positions give copies of its logits)."""
    wl = w.mobilenet_v2_workload(batch=256)
    announce(wl.name)
    x = wl.inputs[0]
    x[100] = x[0]
    x[201] = x[255]
    x[77] = x[130]
    got, kernels = run_on_gpu(device, wl, via="device")
    got = got[0]
    ends = w.mobilenet_v2_workload(batch=8)  # same seed: the same weights
    ends.inputs[0][:4] = x[:4]
    ends.inputs[0][4:] = x[-4:]
    want = oracle_network(ends)
    assert_bit_exact(got[:4], want[:4], "first four images")
    assert_bit_exact(got[-4:], want[4:], "last four images")
    assert np.array_equal(got[100], got[0]) and np.array_equal(got[201], got[255]) and np.array_equal(got[77], got[130])
    assert len(np.unique(got, axis=0)) >= 200  # the logits do depend on the image
    assert "transpose_i8" not in families(kernels)


def test_mobilenet_v2_nchw_declared(device):
    """Same network declared N,C,H,W as the reference emits it: only the input binding is transposed."""
    wl = w.mobilenet_v2_workload(batch=2, resolution=96, classes=100, nhwc=False)
    announce(wl.name, "nchw")
    got, kernels = run_on_gpu(device, wl)
    assert_bit_exact(got[0], oracle_network(wl), wl.name)
    assert families(kernels).count("transpose_i8") == 1 and kernels[0] == "transpose_i8<1>"


def test_graph_replay_matches_oracle_every_time(device):
    """A multi-kernel program on device bindings is captured into a HIP graph on its second dispatch.
    Every replay, with fresh inputs and synchronisations in between, must match the oracle."""
    wl = w.mobilenet_v2_workload(batch=2, resolution=64, classes=40, width=0.5)
    announce(wl.name, "graph replay")
    exe = Executable(device, wl.program.serialize())
    x = wl.inputs[0]
    pin = device.upload(x)
    pout = device.upload(np.zeros((2, 40), dtype=np.int8))
    rng = np.random.default_rng(5)
    for it in range(6):
        if it:
            x[...] = rng.integers(-128, 128, size=x.shape).astype(np.int8)
            runtime.check(runtime.lib().thip_device_h2d(device.handle, pin, x.ctypes.data, x.nbytes))
            device.synchronize()
        if it % 2:
            exe.enqueue_device([pin, pout], [x.nbytes, 80])
            exe.wait()
        else:
            exe.run_device([pin, pout], [x.nbytes, 80])
        got = device.download(pout, (2, 40), np.int8)
        assert_bit_exact(got, oracle_network(wl), "dispatch %d" % it)
    # other buffers: eager again, then a new capture
    pin2 = device.upload(x)
    for it in range(3):
        exe.run_device([pin2, pout], [x.nbytes, 80])
        assert_bit_exact(device.download(pout, (2, 40), np.int8), oracle_network(wl), "second buffer, dispatch %d" % it)
    for ptr in (pin, pin2, pout):
        device.free(ptr)
    exe.close()


def test_program_with_independent_records(device):
    """Three fully_connected records on one input joined by two adds (no path between the first three): the eager
    dispatch, the capture and every replay must give the oracle's bytes, with fresh inputs in between."""
    for M, K, N in [(64, 256, 128), (300, 1024, 512)]:
        wl = w.branches_workload(M, K, N)
        announce(wl.name, "independent records")
        exe = Executable(device, wl.program.serialize())
        x = wl.inputs[0]
        rng = np.random.default_rng(11)
        pin, pout = device.upload(x), device.upload(np.zeros((M, N), dtype=np.int8))
        for it in range(5):
            if it:
                x[...] = rng.integers(-128, 128, size=x.shape).astype(np.int8)
                runtime.check(runtime.lib().thip_device_h2d(device.handle, pin, x.ctypes.data, x.nbytes))
                device.synchronize()
            exe.run_device([pin, pout], [x.nbytes, M * N])
            assert_bit_exact(device.download(pout, (M, N), np.int8), oracle_eval(wl)[0], "dispatch %d" % it)
        exe.close()
        for ptr in (pin, pout):
            device.free(ptr)


def test_full_size_gemm_properties(device):
    """(4096,4096,4096) is too slow for the oracle in a test: check rows the oracle can afford plus a
    structural property (each output row depends on its own input row only)."""
    wl = w.fully_connected_workload(4096, 4096, 4096, realistic=True)
    announce(wl.name)
    got, kernels = run_on_gpu(device, wl, via="device")
    got = got[0]
    from oracle import oracle as orc
    a = dict(wl.attrs)
    wts, sb = a.pop("weights"), a.pop("scale_bias")
    rows = np.r_[0:40, 2000:2040, 4056:4096]
    want = orc.fully_connected(wl.inputs[0][rows], wts, sb, **a)
    assert_bit_exact(got[rows], want, "sampled rows")
    # duplicate input rows give duplicate output rows
    wl.inputs[0][1::2] = wl.inputs[0][0::2]
    got2, _ = run_on_gpu(device, wl, via="device")
    assert np.array_equal(got2[0][1::2], got2[0][0::2]) and np.array_equal(got2[0][0::2], got[0::2])


def test_dispatch_state_validation(device):
    wl = w.add_workload(N=1, H=4, W=4, C=8)
    exe = Executable(device, wl.program.serialize())
    a, b = wl.inputs
    out = np.zeros(a.shape, dtype=np.int8)
    with pytest.raises(ThipError) as e:
        exe.run_host([a, b])  # a binding is missing
    assert e.value.code == runtime.INVALID_ARGUMENT
    with pytest.raises(ThipError) as e:
        exe.run_host([a, b, np.zeros(5, dtype=np.int8)])  # too short
    assert e.value.code == runtime.OUT_OF_RANGE
    st, keep = runtime.make_state([a.ctypes.data, 0, out.ctypes.data], [a.nbytes, b.nbytes, out.nbytes], [0, 0, 0])
    with pytest.raises(ThipError) as e:
        exe.run_state(st)  # NULL binding
    assert e.value.code == runtime.FAILED_PRECONDITION
    # a misaligned device pointer is refused before any launch
    p = device.upload(np.zeros(a.nbytes + 64, dtype=np.int8))
    with pytest.raises(ThipError) as e:
        exe.run_device([p + 1, p, p], [a.nbytes] * 3)
    assert e.value.code == runtime.FAILED_PRECONDITION
    with pytest.raises(ThipError) as e:
        exe.time_device([p, p, p], [a.nbytes] * 3, 0)  # zero iterations
    assert e.value.code == runtime.INVALID_ARGUMENT
    device.free(p)
    # and the executable still works afterwards
    exe.run_host([a, b, out])
    assert_bit_exact(out, oracle_eval(wl)[0], "add after errors")
    exe.close()


def test_event_log_and_timing(device, tmp_path):
    wl = w.maxpool_workload(N=2)
    exe = Executable(device, wl.program.serialize())
    log = tmp_path / "events.csv"
    device.set_event_log(str(log))
    x = wl.inputs[0]
    pin = device.upload(x)
    pout = device.upload(np.zeros(wl.outputs[0][0], dtype=np.int8))
    ms = exe.time_device([pin, pout], [x.nbytes, int(np.prod(wl.outputs[0][0]))], 5)
    device.set_event_log("")
    assert ms > 0
    # the reference's runtime CSV columns, plus the kernel name
    import csv
    rows = list(csv.DictReader(log.open()))
    assert list(rows[0].keys()) == ["dispatch_name", "invocation_id", "action_id", "timestamp_us", "event", "kernel"]
    assert len(rows) == 2 * 5 and [r["event"] for r in rows[:2]] == ["NSS_START_BEGIN", "NSS_START_END"]
    assert all(r["kernel"] == "maxpool2x2_i8" and r["action_id"] == "0" for r in rows)
    assert [int(r["invocation_id"]) for r in rows] == [i // 2 for i in range(10)]
    assert all(int(a["timestamp_us"]) <= int(b["timestamp_us"]) for a, b in zip(rows, rows[1:]))
    # a blocking run on host buffers logs the whole dispatch
    device.set_event_log(str(log))
    host_out = np.zeros(wl.outputs[0][0], dtype=np.int8)
    exe.run_host([x, host_out])
    device.set_event_log("")
    events = [r["event"] for r in csv.DictReader(log.open())]
    assert events == ["DISPATCH_BEGIN", "DISPATCH_SYNC_BINDINGS_IN_BEGIN", "DISPATCH_SYNC_BINDINGS_IN_END", "DISPATCH_EXECUTE_ACTIONS_BEGIN",
                      "NSS_START_BEGIN", "NSS_START_END", "DISPATCH_EXECUTE_ACTIONS_END", "DISPATCH_SYNC_BINDINGS_OUT_BEGIN", "NSS_WAIT_BEGIN",
                      "NSS_WAIT_END", "DISPATCH_SYNC_BINDINGS_OUT_END", "DISPATCH_END"]
    assert_bit_exact(host_out, oracle_eval(wl)[0], "logged run")
    got = device.download(pout, wl.outputs[0][0], np.int8)
    assert_bit_exact(got, oracle_eval(wl)[0], "timed maxpool")
    device.free(pin)
    device.free(pout)
    exe.close()


def test_residual_add_in_the_streaming_epilogue(device, monkeypatch):
    """The add folded behind the requant of the pixel-streaming convolution: both operand orders, ragged rows,
    every accumulator width; and the whole network with and without the folding gives the same bits."""
    # the streaming kernel takes such a convolution on its own from some hundred thousand pixels (the last case); the
    # smaller ones are forced onto it so that every accumulator width of the instantiation with the add runs
    monkeypatch.setenv("THIP_IGEMM_DENSE_VARIANT", "11")
    for kw in [dict(), dict(other_first=True), dict(N=1, H=65, W=66, C=32, O=16), dict(N=3, H=40, W=40, C=144, O=48, other_first=True),
               dict(N=2, H=56, W=56, C=144, O=32), dict(N=4, H=36, W=36, C=64, O=208, other_first=True), dict(N=8, H=28, W=28, C=192, O=64),
               dict(N=130, H=56, W=56, C=96, O=32)]:
        if kw.get("N") == 130:
            monkeypatch.delenv("THIP_IGEMM_DENSE_VARIANT")
        wl = w.pointwise_add_workload(**kw)
        print("[gpu-case]", wl.name, flush=True)
        got, kernels = run_on_gpu(device, wl, via="device")
        assert families(kernels) == ["igemm_stream_i8"] and kernels[0].split(",")[2] == "1", kernels  # the instantiation with the add
        assert_bit_exact(got[0], oracle_eval(wl)[0], wl.name)
    # fewer pixels: the small dense tile adds the residual in its in-register epilogue
    for kw in [dict(N=1, H=8, W=8), dict(N=1, H=14, W=14, C=384, O=64, other_first=True), dict(N=2, H=7, W=7, C=960, O=160), dict(N=1, H=28, W=28, C=192, O=32),
               dict(N=1, H=9, W=7, C=48, O=80, other_first=True), dict(N=8, H=28, W=28, C=192, O=64), dict(N=32, H=14, W=14, C=576, O=96)]:
        wl = w.pointwise_add_workload(**kw)
        print("[gpu-case]", wl.name, flush=True)
        got, kernels = run_on_gpu(device, wl, via="device")
        assert kernels == ["igemm_dense_i8<64,64,2,2,4,4,1,1>"], kernels
        assert_bit_exact(got[0], oracle_eval(wl)[0], wl.name)
    folded, kernels = run_on_gpu(device, w.mobilenet_v2_workload(batch=8), via="device")
    monkeypatch.setenv("THIP_NO_ADD_FUSION", "1")
    apart, kernels_apart = run_on_gpu(device, w.mobilenet_v2_workload(batch=8), via="device")
    assert len(kernels) < len(kernels_apart)
    assert_bit_exact(folded[0], apart[0], "folded vs separate add")
