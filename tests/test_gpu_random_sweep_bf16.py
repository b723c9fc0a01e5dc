"""Seeded random shapes of every bf16 op on the path, through the C-ABI on the GPU, against the oracle.

The counterpart of test_gpu_random_sweep.py for the tolerance rows: fully_connected / matmul / conv2d (GEMMs: at most
1 bf16 ULP per element, or 2^-17 of the sum of |products| where a sum cancels), block-quantized weights expanded in
registers or by the stand-alone kernel, and the ops that repeat the oracle's fp32 operations in the oracle's order
(depthwise, global average pool, add, the expanded weights themselves: bit-exact).  K runs up to 7000 so that the
K split over blocks and its second kernel are drawn too.  The seed is in the test id.
"""
import numpy as np
import pytest

from helpers import assert_bf16_close, assert_bit_exact, oracle_eval, run_on_gpu
from oracle import oracle as orc
from torq_compiler_amd import workloads as w

_mag = lambda bits: np.abs(orc.from_bf16(bits).astype(np.float64))


def _clamp(rng):
    return None if rng.integers(0, 3) else (float(-rng.uniform(0.05, 1.0)), float(rng.uniform(0.05, 1.0)))


def _window(rng, H, W):
    KH, KW = int(rng.integers(1, 4)), int(rng.integers(1, 4))
    pad = tuple(int(v) for v in rng.integers(0, 3, size=4))
    if H + pad[2] + pad[3] < KH:
        KH = 1
    if W + pad[0] + pad[1] < KW:
        KW = 1
    return KH, KW, (int(rng.integers(1, 3)), int(rng.integers(1, 3))), pad


def _fully_connected(device, rng, seed):
    M, K, N = int(rng.integers(1, 90)), 8 * int(rng.integers(1, 900)), int(rng.integers(1, 1400))
    wl = w.fully_connected_bf16_workload(M, K, N, seed=seed, clamp=_clamp(rng))
    got, _ = run_on_gpu(device, wl, via="device" if seed % 2 else "host")
    assert_bf16_close(got[0], oracle_eval(wl)[0], wl.name, magnitude=_mag(wl.inputs[0]) @ _mag(wl.attrs["weights"]).T + np.abs(wl.attrs["bias"]))


def _matmul(device, rng, seed):
    B, M, K, N = int(rng.integers(1, 5)), int(rng.integers(1, 50)), 8 * int(rng.integers(1, 160)), int(rng.integers(1, 300))
    b1, b2 = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    wl = w.matmul_bf16_workload(B, M, K, N, batch1=b1 or not b2, batch2=b2, constant_rhs=bool(rng.integers(0, 2)), seed=seed, bias=float(rng.uniform(-1, 1)))
    got, _ = run_on_gpu(device, wl)
    mag = np.matmul(_mag(wl.inputs[0]), _mag(wl.attrs["input2"])) + abs(float(wl.attrs["bias"][0]))
    assert_bf16_close(got[0], oracle_eval(wl)[0], wl.name, magnitude=np.broadcast_to(mag, got[0].shape))


def _expand_matmul(device, rng, seed):
    block = int(rng.choice([32, 48, 64, 96, 128]))
    M, K, N = int(rng.integers(1, 80)), block * int(rng.integers(1, 40)), int(rng.integers(1, 900))
    wl = w.expand_weights_workload(M=M, K=K, N=N, block=block, fold=bool(rng.integers(0, 4)), clamp=_clamp(rng),
                                   expand_clamp=None if rng.integers(0, 2) else (-0.01, 0.02), bias_pad=int(rng.integers(0, 3)), seed=seed)
    got, _ = run_on_gpu(device, wl, via="device" if seed % 2 else "host")
    w16 = orc.expand_weights(wl.attrs["weights"], wl.attrs["scale"], wl.attrs["qbias"], block_size=wl.attrs["block"],
                             output_min=wl.attrs["expand_min"], output_max=wl.attrs["expand_max"])
    want = oracle_eval(wl)
    assert_bf16_close(got[0], want[0].reshape(got[0].shape), wl.name, magnitude=_mag(wl.inputs[0]) @ _mag(w16) + np.abs(wl.attrs["bias"]).max())
    if not wl.attrs["fold"]:
        assert_bit_exact(got[1], want[1].reshape(got[1].shape), wl.name + ": the expanded weights")


def _conv2d(device, rng, seed):
    H, W = int(rng.integers(1, 30)), int(rng.integers(1, 30))
    KH, KW, stride, pad = _window(rng, H, W)
    nhwc = bool(rng.integers(0, 2))
    wl = w.conv2d_bf16_workload(N=int(rng.integers(1, 4)), H=H, W=W, C=int(rng.integers(1, 70)), O=int(rng.integers(1, 90)), KH=KH, KW=KW, stride=stride,
                                pad=pad, nhwc=nhwc, clamp=_clamp(rng), seed=seed)
    got, _ = run_on_gpu(device, wl)
    # the sum of |products| per output, bounded by |x|max * sum|w| + |bias|
    bound = _mag(wl.attrs["weights"]).reshape(wl.attrs["weights"].shape[0], -1).sum(axis=1) * _mag(wl.inputs[0]).max() + np.abs(wl.attrs["bias"])
    shape = [1, 1, 1, 1]
    shape[3 if nhwc else 1] = -1
    assert_bf16_close(got[0], oracle_eval(wl)[0], wl.name, magnitude=np.broadcast_to(bound.reshape(shape), got[0].shape))


def _depthwise(device, rng, seed):
    H, W = int(rng.integers(1, 40)), int(rng.integers(1, 40))
    KH, KW, stride, pad = _window(rng, H, W)
    wl = w.conv2d_bf16_workload(depthwise=True, N=int(rng.integers(1, 4)), H=H, W=W, C=int(rng.integers(1, 200)), KH=KH, KW=KW, stride=stride, pad=pad,
                                nhwc=bool(rng.integers(0, 2)), clamp=_clamp(rng), seed=seed)
    got, _ = run_on_gpu(device, wl)
    assert_bit_exact(got[0], oracle_eval(wl)[0], wl.name)


def _avg_pool(device, rng, seed):
    wl = w.avg_pool2d_bf16_workload(N=int(rng.integers(1, 70)), H=int(rng.integers(1, 16)), W=int(rng.integers(1, 16)), C=int(rng.integers(1, 1400)),
                                    weight=None if rng.integers(0, 2) else float(rng.uniform(0.001, 1)), clamp=_clamp(rng), seed=seed)
    got, _ = run_on_gpu(device, wl)
    assert_bit_exact(got[0], oracle_eval(wl)[0], wl.name)


def _add(device, rng, seed):
    shape = tuple(int(v) for v in rng.integers(1, 40, size=int(rng.integers(1, 5))))
    wl = w.add_bf16_workload(shape, float(rng.uniform(-2, 2)), float(rng.uniform(-2, 2)), float(rng.uniform(-1, 1)), clamp=_clamp(rng), seed=seed)
    got, _ = run_on_gpu(device, wl)
    assert_bit_exact(got[0], oracle_eval(wl)[0], wl.name)


FAMILIES = [("fully_connected", _fully_connected, 40), ("matmul", _matmul, 30), ("expand_matmul", _expand_matmul, 30), ("conv2d", _conv2d, 30),
            ("depthwise", _depthwise, 25), ("avg_pool", _avg_pool, 20), ("add", _add, 15)]
SWEEP = [(name, run, 5000000 + 1000 * f + i) for f, (name, run, count) in enumerate(FAMILIES) for i in range(count)]


@pytest.mark.gpu
@pytest.mark.parametrize("name,run,seed", SWEEP, ids=["%s-%d" % (c[0], c[2]) for c in SWEEP])
def test_random_bf16_shape(device, name, run, seed):
    print("[gpu-case] bf16", name, "seed", seed, flush=True)
    run(device, np.random.default_rng(seed), seed)


@pytest.mark.gpu
def test_random_bf16_tolerance_tally(device):
    """Of the elements this sweep compared under the tolerance, how many were beyond one bf16 step and admitted by the
    cancellation bound: printed, and a small minority."""
    import helpers
    mine = [t for t in helpers.BF16_TALLY if t[0].startswith(("fcbf16", "matmulbf16", "expandmm", "convbf16")) and not t[0].endswith("(gpu)")]
    if not mine:
        pytest.skip("the sweep did not run in this process")
    compared, widened = sum(n for _, n, _ in mine), sum(k for _, _, k in mine)
    print("[bf16-tolerance] random sweep: %d of %d elements (%.4f %%) in %d comparisons beyond one step" % (widened, compared, 100.0 * widened / compared, len(mine)), flush=True)
    assert widened <= compared * 1e-4
