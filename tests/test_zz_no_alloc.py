"""thip_executable_enqueue_noalloc: the dispatch that allocates nothing, against thip_executable_enqueue.

The kernels with scratch memory are the bf16 fully_connected / matmul records whose K is split over blocks (partial
sums).  The no-allocation entry point takes that memory from the library's static device array,
which every call on the GPU shares and which keeps the last call's contents: two calls in a row, the second on a
smaller problem, must each give exactly what the ordinary entry point gives.
"""
import sys

import numpy as np
import pytest

import desc_interp
from helpers import assert_bf16_close, assert_bit_exact, families, oracle_eval
from oracle import oracle as orc
from torq_compiler_amd import Executable, Program, ThipError, runtime, workloads as w

pytestmark = pytest.mark.gpu


def _split_of(wl):
    d = desc_interp.Descriptor(wl.program.serialize())
    return [int(o["w0"]) for o in d.ops if int(o["kind"]) == desc_interp.K_FC_BF16]


def _both_ways(device, wl):
    """Outputs of the ordinary enqueue and of the no-allocation enqueue on the same device buffers."""
    print("[gpu-case]", wl.name, "enqueue vs enqueue_noalloc", flush=True)
    sys.stdout.flush()
    exe = Executable(device, wl.program.serialize())
    shape, dt = wl.outputs[0]
    ins = [device.upload(a) for a in wl.inputs]
    lens = [a.nbytes for a in wl.inputs] + [int(np.prod(shape)) * np.dtype(dt).itemsize]
    results = []
    try:
        for noalloc in (False, True, True):
            pout = device.upload(np.full(shape, 0x55, dtype=dt))
            (exe.enqueue_device_noalloc if noalloc else exe.enqueue_device)(ins + [pout], lens)
            exe.wait()
            results.append(device.download(pout, shape, dt))
            device.free(pout)
        kernels = exe.op_kernels()
    finally:
        exe.close()
        for p in ins:
            device.free(p)
    return results, kernels


def test_noalloc_matches_enqueue_twice_in_a_row(device):
    f = lambda bits: np.abs(orc.from_bf16(bits).astype(np.float64))
    # a long K over a handful of output tiles: K split 9 ways; then a smaller problem, split 5 ways
    for (M, K, N), split in [((1, 6912, 256), 9), ((3, 4096, 128), 5)]:
        wl = w.fully_connected_bf16_workload(M, K, N)
        assert _split_of(wl) == [split], "the workload must take the K-split kernels (scratch: partial sums)"
        (plain, first, again), kernels = _both_ways(device, wl)
        assert families(kernels) == ["fc_bf16"]
        assert_bit_exact(first, plain, wl.name + ": no-allocation entry point against thip_executable_enqueue")
        assert_bit_exact(again, plain, wl.name + ": second call on the same scratch")
        mag = f(wl.inputs[0]) @ f(wl.attrs["weights"]).T + np.abs(wl.attrs["bias"])
        assert_bf16_close(first, oracle_eval(wl)[0], wl.name, magnitude=mag)


def test_noalloc_without_scratch_and_on_a_whole_network(device):
    """Programs whose kernels use no scratch run unchanged: an int8 GEMM, and a small mobile network."""
    for wl in [w.fully_connected_workload(64, 256, 128, realistic=True), w.mobilenet_v2_workload(batch=2, resolution=64, classes=40, width=0.5)]:
        (plain, first, again), _ = _both_ways(device, wl)
        assert_bit_exact(first, plain, wl.name)
        assert_bit_exact(again, plain, wl.name)


def test_noalloc_refuses_what_does_not_fit_and_host_bindings(device):
    # four K-split linears of 16 tiles x 9 slices each: 2.25 MiB of partial sums, the array holds 2 MiB
    rng = np.random.default_rng(3)
    p = Program()
    x = p.binding(0, (32, 6912), np.uint16)
    weights = [w.to_bf16(rng.standard_normal((512, 6912)) / 83.0) for _ in range(4)]
    for i, wt in enumerate(weights):
        p.fully_connected(x, wt, np.zeros(512, dtype=np.float32), init=p.binding(1 + i, (32, 512), np.uint16), output_zp=0, shift_factor=0,
                          input_zp=0, output_min=w.NO_CLAMP[0], output_max=w.NO_CLAMP[1])
    blob = p.serialize()
    assert [int(o["w0"]) for o in desc_interp.Descriptor(blob).ops] == [9, 9, 9, 9]
    exe = Executable(device, blob)
    xin = w.to_bf16(rng.standard_normal((32, 6912)))
    ptrs = [device.upload(xin)] + [device.upload(np.zeros((32, 512), dtype=np.uint16)) for _ in range(4)]
    lens = [xin.nbytes] + [32 * 512 * 2] * 4
    try:
        with pytest.raises(ThipError) as err:
            exe.enqueue_device_noalloc(ptrs, lens)
        assert err.value.code == runtime.RESOURCE_EXHAUSTED and "scratch" in err.value.message
        exe.enqueue_device(ptrs, lens)  # the ordinary entry point runs it from the executable's own intermediates
        exe.wait()
        got = device.download(ptrs[1], (32, 512), np.uint16)
        want = orc.fully_connected_bf16(xin, weights[0], np.zeros(512, dtype=np.float32))
        f = lambda bits: np.abs(orc.from_bf16(bits).astype(np.float64))
        assert_bf16_close(got, want, "first linear", magnitude=f(xin) @ f(weights[0]).T)
    finally:
        exe.close()
        for ptr in ptrs:
            device.free(ptr)
    # host pointers would need staging buffers, i.e. an allocation
    wl = w.fully_connected_bf16_workload(1, 6912, 256)
    exe = Executable(device, wl.program.serialize())
    out = np.zeros((1, 256), dtype=np.uint16)
    st, keep = runtime.make_state([wl.inputs[0].ctypes.data, out.ctypes.data], [wl.inputs[0].nbytes, out.nbytes], [0, 0])
    import ctypes
    code = runtime.lib().thip_executable_enqueue_noalloc(exe._h, ctypes.byref(st))
    exe.close()
    assert code == runtime.FAILED_PRECONDITION
