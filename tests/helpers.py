"""Shared helpers of the test-suite: run a workload through the C-ABI, evaluate it with the oracle."""
import numpy as np

from oracle.programs import (BF16_TALLY, assert_bf16_close, assert_bit_exact, bf16_ordered,  # noqa: F401  (re-exported)
                             eval_network as oracle_network, eval_workload as oracle_eval)


def run_on_gpu(device, wl, via="host"):
    """Serialises the workload's program, loads it and runs one dispatch; returns the outputs."""
    import torq_compiler_amd as thip

    blob = wl.program.serialize()
    exe = thip.Executable(device, blob)
    outs = [np.full(shape, 0x55, dtype=dt) for shape, dt in wl.outputs]
    try:
        if via == "host":
            exe.run_host(list(wl.inputs) + outs)
        else:
            ptrs = [device.upload(a) for a in wl.inputs] + [device.upload(o) for o in outs]
            lens = [a.nbytes for a in wl.inputs] + [o.nbytes for o in outs]
            exe.run_device(ptrs, lens)
            n_in = len(wl.inputs)
            outs = [device.download(ptrs[n_in + i], o.shape, o.dtype) for i, o in enumerate(outs)]
            for p in ptrs:
                device.free(p)
        return outs, exe.op_kernels()
    finally:
        exe.close()


def families(kernels):
    """Kernel names without their template arguments: "maxpool_i8<16>" -> "maxpool_i8"."""
    return [k.split("<")[0] for k in kernels]


