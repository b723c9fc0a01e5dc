"""Seeded random geometries of every op on the path, through the C-ABI on the GPU, bit-exact against the oracle.

The fixed cases of test_gpu_parity.py are the benchmark shapes and the geometries the reference's own tests use; this
sweep draws what nobody thought of: odd frames, windows that hang over the border on one side only, strides up to 4,
channel counts around the vector widths (1, 3, 4, 15, 16, 17, 24, 33 ...), clamps narrower than the type, zero points of
either sign, requant shifts on both sides of the 32-bit tails.  Every case is small enough for the oracle to finish in
milliseconds; the seed is in the test id, so a failure names its case.  The emitter is free to pick any kernel: the
test asserts only that some kernel of the op's family ran, and the result.
"""
import numpy as np
import pytest

from helpers import assert_bit_exact, families, oracle_eval, oracle_network, run_on_gpu
from torq_compiler_amd import workloads as w

CHANNELS = [1, 3, 4, 8, 15, 16, 17, 24, 32, 33, 48, 64, 96, 144]


def _window(rng, H, W):
    KH, KW = int(rng.integers(1, min(5, H) + 1)), int(rng.integers(1, min(5, W) + 1))
    pad = [int(rng.integers(0, KW)), int(rng.integers(0, KW)), int(rng.integers(0, KH)), int(rng.integers(0, KH))]  # l, r, t, b < window
    stride = (int(rng.integers(1, 5)), int(rng.integers(1, 5)))
    return KH, KW, tuple(pad), stride


def _clamp(rng, zp):
    lo = int(rng.choice([-128, -128, zp, -100]))
    hi = int(rng.choice([127, 127, 127, 90]))
    return min(lo, hi), max(lo, hi)


def _conv(seed):
    rng = np.random.default_rng(seed)
    H, W = int(rng.integers(1, 24)), int(rng.integers(1, 24))
    KH, KW, pad, stride = _window(rng, H, W)
    zp = int(rng.integers(-128, 128))
    lo, hi = _clamp(rng, zp)
    return w.conv2d_workload(N=int(rng.integers(1, 4)), H=H, W=W, C=int(rng.choice(CHANNELS)), O=int(rng.choice(CHANNELS)), KH=KH, KW=KW,
                             stride=stride, pad=pad, input_zp=int(rng.integers(-128, 128)), output_zp=zp, output_min=lo, output_max=hi,
                             realistic=bool(rng.integers(0, 4)), nhwc=bool(rng.integers(0, 2)), seed=seed)


def _depthwise(seed):
    rng = np.random.default_rng(seed)
    H, W = int(rng.integers(1, 30)), int(rng.integers(1, 30))
    if rng.integers(0, 2):  # the 3x3 kernels' territory: stride 1 or 2, C a multiple of 16
        H, W = max(H, 3), max(W, 3)
        KH = KW = 3
        s = int(rng.integers(1, 3))
        stride, pad = (s, s), tuple(int(v) for v in rng.integers(0, 2, size=4))
        C = int(rng.choice([16, 32, 48, 96, 144]))
    else:
        KH, KW, pad, stride = _window(rng, H, W)
        C = int(rng.choice(CHANNELS))
    zp = int(rng.integers(-128, 128))
    lo, hi = _clamp(rng, zp)
    shift = None if rng.integers(0, 2) else int(rng.choice([0, 1, 12, 24, 31, 32, 33, 40, 62]))
    return w.depthwise_workload(N=int(rng.integers(1, 4)), H=H, W=W, C=C, KH=KH, KW=KW, stride=stride, pad=pad, input_zp=int(rng.integers(-128, 128)),
                                output_zp=zp, output_min=lo, output_max=hi, realistic=True, nhwc=bool(rng.integers(0, 2)), seed=seed, shift=shift)


def _fully_connected(seed):
    rng = np.random.default_rng(seed)
    M = int(rng.choice([1, 1, 2, 5, 16, 17, 33, 64, 130]))
    K = int(rng.choice([1, 3, 16, 24, 61, 64, 100, 128, 200, 512]))
    N = int(rng.choice([1, 7, 16, 31, 32, 40, 97, 128, 200]))
    zp = int(rng.integers(-128, 128))
    lo, hi = _clamp(rng, zp)
    shift = None if rng.integers(0, 2) else int(rng.choice([0, 6, 31, 32, 33, 45, 46, 62]))
    return w.fully_connected_workload(M, K, N, realistic=bool(rng.integers(0, 2)), output_zp=zp, output_min=lo, output_max=hi, seed=seed, shift=shift)


def _matmul(seed):
    rng = np.random.default_rng(seed)
    b1, b2 = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    B = int(rng.integers(1, 4)) if (b1 or b2) else 1
    out = [np.int8, np.int16, np.int32][int(rng.integers(0, 3))]
    constant = bool(rng.integers(0, 2)) and not b2
    scale, shift = [(1, 0), (3, 2), (1 << 20, 27), (77, 9)][int(rng.integers(0, 4))]
    return w.matmul_workload(B, int(rng.choice([1, 4, 9, 33])), int(rng.choice([1, 8, 16, 37, 64, 128])), int(rng.choice([1, 5, 16, 40, 64])),
                             batch1=b1, batch2=b2, constant_rhs=constant, out_dtype=out, bias=int(rng.integers(-50, 50)), scale=scale, shift=shift,
                             output_zp=int(rng.integers(-5, 6)), seed=seed)


def _maxpool(seed):
    rng = np.random.default_rng(seed)
    H, W = int(rng.integers(1, 30)), int(rng.integers(1, 30))
    KH, KW, pad, stride = _window(rng, H, W)
    if rng.integers(0, 3) == 0 and H >= 2 and W >= 2:  # the 2x2 stride-2 kernel's territory
        KH, KW, pad, stride = 2, 2, (0, int(W % 2), 0, int(H % 2)), (2, 2)
    return w.maxpool_workload(N=int(rng.integers(1, 4)), H=H, W=W, C=int(rng.choice(CHANNELS)), kernel=(KH, KW), stride=stride, pad=pad,
                              input_zp=int(rng.choice([-128, -128, 0, 17])), nhwc=bool(rng.integers(0, 2)), seed=seed)


def _avgpool(seed):
    rng = np.random.default_rng(seed)
    return w.avgpool_workload(N=int(rng.integers(1, 5)), H=int(rng.integers(1, 20)), W=int(rng.integers(1, 20)), C=int(rng.choice(CHANNELS + [1280])),
                              input_zp=int(rng.integers(-128, 128)), output_zp=int(rng.integers(-20, 20)), seed=seed)


def _add(seed):
    rng = np.random.default_rng(seed)
    return w.add_workload(N=int(rng.integers(1, 4)), H=int(rng.integers(1, 20)), W=int(rng.integers(1, 20)), C=int(rng.choice(CHANNELS)),
                          zp0=int(rng.integers(-128, 128)), zp1=int(rng.integers(-128, 128)), m0=float(rng.uniform(0.05, 3.0)), m1=float(rng.uniform(0.05, 3.0)),
                          output_zp=int(rng.integers(-128, 128)), seed=seed)


def _conv_ring(seed, channels=(64, 64, 128, 192), images=(3, 6), extent=(30, 50)):
    """A multiple of 16 channels, 64 or more, and at least 2048 output pixels: the ring kernel's window addressing."""
    rng = np.random.default_rng(seed)
    KH, KW = int(rng.integers(1, 5)), int(rng.integers(1, 5))
    stride = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
    H, W = int(rng.integers(*extent)) * stride[0], int(rng.integers(*extent)) * stride[1]
    pad = (int(rng.integers(0, KW)), int(rng.integers(0, KW)), int(rng.integers(0, KH)), int(rng.integers(0, KH)))
    zp = int(rng.integers(-128, 128))
    lo, hi = _clamp(rng, zp)
    return w.conv2d_workload(N=int(rng.integers(*images)), H=H, W=W, C=int(rng.choice(channels)), O=int(rng.choice([32, 48, 64, 72, 96, 160, 272])), KH=KH, KW=KW,
                             stride=stride, pad=pad, input_zp=int(rng.integers(-128, 128)), output_zp=zp, output_min=lo, output_max=hi,
                             realistic=bool(rng.integers(0, 4)), nhwc=bool(rng.integers(0, 2)), seed=seed)


def _conv_ring16(seed):
    """Channel counts that are not whole k-tiles: k-tiles straddle taps and the last one reaches beyond K."""
    return _conv_ring(seed, channels=(80, 96, 112, 144, 160, 176, 208, 240, 272))


def _conv_ring_few(seed):
    """Fewer channels than a k-tile over at least 20 000 output pixels: several taps per k-tile."""
    return _conv_ring(seed, channels=(16, 32, 48), images=(10, 15), extent=(50, 60))


SWEEP = ([("conv2d", _conv, s, {"igemm_i8", "igemm_dense_i8", "igemm_stream_i8", "igemm_dense_conv_i8"}) for s in range(5000, 5200)] +
         [("conv2d_ring", _conv_ring, s, {"igemm_dense_conv_i8"}) for s in range(5500, 5530)] +
         [("conv2d_ring16", _conv_ring16, s, {"igemm_dense_conv_i8"}) for s in range(5600, 5640)] +
         [("conv2d_ring_few", _conv_ring_few, s, {"igemm_dense_conv_i8"}) for s in range(5700, 5730)] +
         [("depthwise", _depthwise, s, {"depthwise3x3_strip_i8", "depthwise3x3_tile_i8", "depthwise3x3_dot4_i8", "depthwise_i8"}) for s in range(6000, 6200)] +
         [("fully_connected", _fully_connected, s, {"igemm_i8", "igemm_dense_i8", "igemm_stream_i8", "fc_skinny", "fc_skinny_mfma"}) for s in range(7000, 7150)] +
         [("matmul", _matmul, s, {"igemm_i8", "igemm_dense_i8", "igemm_stream_i8", "fc_skinny", "fc_skinny_mfma"}) for s in range(8000, 8100)] +
         [("maxpool", _maxpool, s, {"maxpool_i8", "maxpool2x2_i8"}) for s in range(9000, 9150)] +
         [("avgpool", _avgpool, s, {"avgpool_i8"}) for s in range(10000, 10050)] +
         [("add", _add, s, {"add_i8"}) for s in range(11000, 11050)])


@pytest.mark.gpu
@pytest.mark.parametrize("op,make,seed,allowed", SWEEP, ids=["%s-%d" % (c[0], c[2]) for c in SWEEP])
def test_random_geometry(device, op, make, seed, allowed):
    wl = make(seed)
    print("[gpu-case]", op, seed, wl.name, flush=True)
    got, kernels = run_on_gpu(device, wl, via="host" if seed % 2 else "device")
    want = oracle_eval(wl)
    for g, e in zip(got, want):
        assert_bit_exact(g, e, "%s seed %d (%s)" % (op, seed, wl.name))
    main = [k for k in families(kernels) if k != "transpose_i8"]
    assert main and set(main) <= allowed, (kernels, allowed)


# Whole programs: the mobile network at other widths, resolutions, batch sizes and seeds.  The channel counts move with
# the width (8 .. 416 per bottleneck, some multiples of 16 and some not), so the emitter's layout decisions (channel
# padding of intermediates, which adds fold into a convolution's epilogue, which kernel each layer gets) all change.
NETWORKS = [dict(width=wd, resolution=r, batch=b, nhwc=n, seed=2000 + i)
            for i, (wd, r, b, n) in enumerate([(0.25, 32, 1, True), (0.25, 64, 3, False), (0.35, 32, 2, True), (0.5, 64, 1, True), (0.5, 32, 5, False),
                                               (0.75, 32, 1, False), (0.75, 96, 2, True), (1.0, 32, 4, True), (1.0, 64, 1, False), (1.3, 32, 2, True),
                                               (1.4, 64, 1, True), (0.35, 96, 1, False)])]


@pytest.mark.gpu
@pytest.mark.parametrize("kw", NETWORKS, ids=lambda kw: "w%s-r%d-b%d-%s" % (kw["width"], kw["resolution"], kw["batch"], "nhwc" if kw["nhwc"] else "nchw"))
def test_random_network(device, kw):
    wl = w.mobilenet_v2_workload(classes=37, **kw)
    print("[gpu-case]", wl.name, kw, flush=True)
    got, kernels = run_on_gpu(device, wl, via="device")
    assert_bit_exact(got[0], oracle_network(wl), wl.name)
    assert len(kernels) >= 50


def test_networks_through_the_descriptor_interpreter():
    import desc_interp
    for kw in NETWORKS[:6]:
        wl = w.mobilenet_v2_workload(classes=37, **kw)
        outs = [np.zeros(s, dtype=dt) for s, dt in wl.outputs]
        desc_interp.run(wl.program.serialize(), list(wl.inputs) + outs)
        assert_bit_exact(outs[0], oracle_network(wl), wl.name)


def test_sweep_through_the_descriptor_interpreter():
    """The same cases without a GPU: what the emitter writes for each of them, evaluated by the numpy descriptor
    interpreter, must already equal the oracle (so a GPU failure of the sweep points at a kernel, not at the emitter)."""
    import desc_interp
    for op, make, seed, _ in SWEEP:
        wl = make(seed)
        outs = [np.zeros(s, dtype=dt) for s, dt in wl.outputs]
        desc_interp.run(wl.program.serialize(), list(wl.inputs) + outs)
        assert_bit_exact(outs[0], oracle_eval(wl)[0], "%s seed %d (%s)" % (op, seed, wl.name))
