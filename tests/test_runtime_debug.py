"""Run-side debugging aids on the GPU: buffer dumps (the role of the reference's runtime/driver/TorqDump.cc) and the
bounded wait (runtime/torq_hw/src/TorqHw.cpp:172-186: a wait that exceeds its timeout becomes an INTERNAL status)."""
import os
import sys

import numpy as np
import pytest

from helpers import assert_bit_exact, oracle_eval, oracle_network
from torq_compiler_amd import Executable, ThipError, runtime, workloads as w

pytestmark = pytest.mark.gpu


def test_buffer_and_binding_dumps(device, tmp_path, monkeypatch):
    """Every kernel record's output, dumped as .npy, against the oracle's tensor for that layer (a small mobile network
    with the residual adds and the channel padding left out of the records, so that record i is layer i), and the
    bindings of the blocking dispatch under the reference's file names."""
    monkeypatch.setenv("THIP_NO_ADD_FUSION", "1")
    monkeypatch.setenv("THIP_NO_CHANNEL_PAD", "1")
    wl = w.mobilenet_v2_workload(batch=2, resolution=64, classes=40, width=0.5)
    print("[gpu-case]", wl.name, "with dumps", flush=True)
    sys.stdout.flush()
    tensors = oracle_network(wl, return_all=True)
    io_dir, buf_dir = str(tmp_path / "io"), str(tmp_path / "buffers")
    wl.program.set_name("mbv2_small")  # the directory the dumps go to
    exe = Executable(device, wl.program.serialize())
    out = np.zeros(wl.outputs[0][0], dtype=np.int8)
    device.set_dump_dirs(io_dir, buf_dir)
    try:
        exe.run_host([wl.inputs[0], out])
    finally:
        device.set_dump_dirs(None, None)
    kernels = exe.op_kernels()
    exe.close()
    assert_bit_exact(out, tensors[-1], "logits with dumps on")
    assert len(kernels) == len(tensors) - 1
    base = os.path.join(buf_dir, "mbv2_small")
    for i in range(len(kernels)):
        files = os.listdir(os.path.join(base, "action%d" % i))
        assert len(files) == 1 and files[0].startswith("buffer") and files[0].endswith(".npy"), files
        got = np.load(os.path.join(base, "action%d" % i, files[0]), allow_pickle=False)
        want = tensors[i + 1]
        assert got.dtype == np.int8 and got.size == want.size, (i, kernels[i], got.shape, want.shape)
        assert_bit_exact(got.reshape(want.shape), want, "record %d (%s)" % (i, kernels[i]))
    index = open(os.path.join(base, "buffers.csv")).read().splitlines()
    assert index[0].startswith("id;type;shape;strides;address;size;allocation_action;last_use_action;deallocation_action")
    assert len(index) == 1 + len(kernels) and index[-1].startswith("binding1;BINDING;2x40xi8;")
    io = os.path.join(io_dir, "mbv2_small")
    assert np.array_equal(np.fromfile(os.path.join(io, "npu.in.host_binding.0.torq_binding.0.bin"), dtype=np.int8), wl.inputs[0].reshape(-1))
    assert np.array_equal(np.fromfile(os.path.join(io, "npu.out.host_binding.1.torq_binding.1.bin"), dtype=np.int8), out.reshape(-1))
    # dumps off again: nothing new is written
    before = sorted(os.listdir(base))
    exe = Executable(device, w.add_workload(N=1, H=8, W=8, C=24).program.serialize())
    exe.close()
    assert sorted(os.listdir(base)) == before


def test_wait_timeout_becomes_a_status(device):
    """A wait that exceeds its limit returns INTERNAL and abandons the executable; the kernels themselves finish
    normally (the limit is what is made tiny, not the work made endless) and the process carries on."""
    wl = w.fully_connected_workload(4096, 4096, 4096)
    print("[gpu-case]", wl.name, "wait timeout", flush=True)
    sys.stdout.flush()
    exe = Executable(device, wl.program.serialize())
    ptrs = [device.upload(wl.inputs[0]), device.upload(np.zeros((4096, 4096), dtype=np.int8))]
    lens = [wl.inputs[0].nbytes, 4096 * 4096]
    exe.run_device(ptrs, lens)  # within the default limit
    exe.set_wait_timeout(1)
    for _ in range(400):  # tens of milliseconds of queued work
        exe.enqueue_device(ptrs, lens)
    with pytest.raises(ThipError) as err:
        exe.wait()
    assert err.value.code == runtime.INTERNAL and "did not finish within 1 ms" in err.value.message
    with pytest.raises(ThipError) as err:
        exe.enqueue_device(ptrs, lens)
    assert err.value.code == runtime.FAILED_PRECONDITION
    with pytest.raises(ThipError) as err:
        exe.run_device(ptrs, lens)
    assert err.value.code == runtime.FAILED_PRECONDITION
    device.synchronize()  # the queued kernels run to their normal end
    got = device.download(ptrs[1], (4096, 4096), np.int8)
    exe.close()
    for p in ptrs:
        device.free(p)
    # the device is as usable as before
    other = w.fully_connected_workload(64, 256, 128, realistic=True)
    exe2 = Executable(device, other.program.serialize())
    res = np.zeros((64, 128), dtype=np.int8)
    exe2.run_host([other.inputs[0], res])
    exe2.close()
    assert_bit_exact(res, oracle_eval(other)[0], other.name)
    assert got.shape == (4096, 4096)


def test_dispatches_from_two_threads(device):
    """The run-side contract of the reference (one dispatch at a time per executable behind a mutex, callers on any
    thread: runtime/driver/TorqExecutable.cc:1045): two threads dispatch two executables at the same time, then both
    dispatch the same one; every result is the oracle's."""
    import threading
    wls = [w.conv2d_workload(N=2, H=28, W=28, C=32, O=64, realistic=True), w.branches_workload(64, 256, 128)]
    wants = [oracle_eval(wl)[0] for wl in wls]
    exes = [Executable(device, wl.program.serialize()) for wl in wls]
    print("[gpu-case] two threads,", wls[0].name, "and", wls[1].name, flush=True)
    sys.stdout.flush()
    errors = []

    def worker(which, rounds):
        try:
            wl, want, exe = wls[which], wants[which], exes[which]
            for _ in range(rounds):
                out = np.zeros(wl.outputs[0][0], dtype=np.int8)
                exe.run_host(list(wl.inputs) + [out])   # blocking; the library call runs without the interpreter lock
                if not np.array_equal(out, want):
                    errors.append("%s differs" % wl.name)
                    return
        except Exception as ex:  # reported by the main thread
            errors.append(repr(ex))

    try:
        for pair in ((0, 1), (0, 0), (1, 1)):
            threads = [threading.Thread(target=worker, args=(which, 40)) for which in pair]
            for t in threads:
                t.start()
            for t in threads:
                t.join(timeout=100)
            assert not any(t.is_alive() for t in threads), "a dispatching thread did not finish"
            assert not errors, errors
    finally:
        for exe in exes:
            exe.close()
