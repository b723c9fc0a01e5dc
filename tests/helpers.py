"""Shared helpers of the test-suite: run a workload through the C-ABI, evaluate it with the oracle."""
import numpy as np

from oracle import oracle as orc


def oracle_eval(wl):
    """Expected outputs of a single-op workload, computed by the CPU oracle."""
    a = dict(wl.attrs)
    kind = wl.name.split("_")[0]
    x = wl.inputs[0]
    if kind == "conv2d":
        layout = orc.NHWC if a.pop("nhwc") else orc.NCHW
        w, sb = a.pop("weights"), a.pop("scale_bias")
        return [orc.conv2d(x, w, sb, layout=layout, **a)]
    if kind == "depthwise":
        layout = orc.NHWC if a.pop("nhwc") else orc.NCHW
        w, sb = a.pop("weights"), a.pop("scale_bias")
        return [orc.depthwise_conv2d(x, w, sb, layout=layout, **a)]
    if kind == "fully":
        w, sb = a.pop("weights"), a.pop("scale_bias")
        return [orc.fully_connected(x, w, sb, **a)]
    if kind == "maxpool":
        layout = orc.NHWC if a.pop("nhwc") else orc.NCHW
        return [orc.maxpool2d(x, layout=layout, **a)]
    if kind == "avgpool":
        sb = a.pop("scale_bias")
        a.pop("input_zp")
        return [orc.avg_pool2d(x, sb, **a)]
    if kind == "add":
        w, sb = a.pop("weights"), a.pop("scale_bias")
        return [orc.add(wl.inputs[0], wl.inputs[1], w, sb, **a)]
    raise ValueError(wl.name)


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


def assert_bit_exact(got, want, what=""):
    assert got.shape == want.shape and got.dtype == want.dtype, (what, got.shape, want.shape, got.dtype, want.dtype)
    if not np.array_equal(got, want):
        bad = np.argwhere(got != want)
        first = tuple(bad[0])
        raise AssertionError("%s: %d of %d elements differ; first at %s: got %d want %d"
                             % (what, len(bad), got.size, first, int(got[first]), int(want[first])))


def oracle_network(wl, return_all=False):
    """Replays a network workload (wl.attrs['layers']) layer by layer with the CPU oracle, N,H,W,C."""
    layers = wl.attrs["layers"]
    x = wl.inputs[0]
    if not wl.attrs["nhwc"]:
        x = np.ascontiguousarray(x.transpose(0, 2, 3, 1))
    tensors = [x]
    for L in layers:
        src = [tensors[i] for i in L.inputs]
        a = dict(L.attrs)
        if L.op == "conv2d":
            t = orc.conv2d(src[0], L.weights, L.scale_bias, layout=orc.NHWC, **a)
        elif L.op == "depthwise_conv2d":
            t = orc.depthwise_conv2d(src[0], L.weights, L.scale_bias, layout=orc.NHWC, **a)
        elif L.op == "add":
            t = orc.add(src[0], src[1], L.weights, L.scale_bias, **a)
        elif L.op == "avg_pool2d":
            a.pop("input_zp")
            t = orc.avg_pool2d(src[0], L.scale_bias, **a)
        elif L.op == "fully_connected":
            t = orc.fully_connected(src[0].reshape(src[0].shape[0], -1), L.weights, L.scale_bias, **a)
        else:
            raise ValueError(L.op)
        tensors.append(t)
    return tensors if return_all else tensors[-1]
