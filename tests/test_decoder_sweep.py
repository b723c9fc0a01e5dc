"""Drawn, not listed: grouped linears on block-quantized weights and attention steps of random shape -- rows 1 .. 32,
K any multiple of 128 up to 2048 (and the decoder's 6912), every grouping, block size, clamp and zero-point choice --
through the descriptor interpreter on the CPU and through the C-ABI on the GPU, each op checked on the inputs the run
gave it (<= 1 bf16 ULP, the adds bit-exactly)."""
import numpy as np
import pytest

import desc_interp
import torq_compiler_amd as thip
from oracle import programs as prog
from torq_compiler_amd import workloads as w


def draw_linear(seed):
    rng = np.random.default_rng(7000 + seed)
    mode = ["single", "concat", "pair", "pair_hidden", "residual", "residual_first"][int(rng.integers(0, 6))]
    K = 128 * int(rng.integers(1, 17)) if rng.integers(0, 8) else 6912
    blocks = [b for b in (128, 256, 384, 512, K) if K % b == 0]
    case = dict(mode=mode, M=int(rng.integers(1, 33)), K=K, block=int(blocks[int(rng.integers(0, len(blocks)))]),
                N=K if mode.startswith("residual") else 16 * int(rng.integers(1, 25 if K <= 2048 else 5)) * (2 if mode == "concat" else 1),
                zero_points=bool(rng.integers(0, 2)), seed=1050 + seed)
    if mode.startswith("residual") and K > 2048:
        case.update(K=1152, N=1152, block=128 if case["block"] not in (128, 384, 1152) else case["block"])
    if rng.integers(0, 3) == 0:
        case["clamp"] = (-float(rng.uniform(0.1, 1.0)), float(rng.uniform(0.1, 1.0)))
    if rng.integers(0, 4) == 0:
        case["expand_clamp"] = (-float(rng.uniform(0.005, 0.05)), float(rng.uniform(0.005, 0.05)))
    return case


def draw_attention(seed):
    rng = np.random.default_rng(9000 + seed)
    case = dict(B=int(rng.integers(1, 6)), H=int(rng.integers(1, 33)), D=8 * int(rng.integers(1, 40)), T=int(rng.integers(1, 300)),
                D2=int(rng.integers(1, 200)), seed=1045 + seed)
    case["T"] = 8 * max(1, case["T"] // 8)  # the second product's K
    if rng.integers(0, 3) == 0:
        case.update(bias=(float(rng.uniform(-0.5, 0.5)), float(rng.uniform(-0.5, 0.5))), clamp1=(-1.0, 1.5), clamp2=(-0.75, 0.5))
    return case


def _exact(got, want, what, magnitude=None):
    prog.assert_bit_exact(got, want, what)


@pytest.mark.parametrize("seed", range(40))
def test_drawn_grouped_linear_records(seed):
    wl = w.grouped_linear_workload(**draw_linear(seed))
    blob = wl.program.serialize()
    kinds = [int(o["kind"]) for o in desc_interp.Descriptor(blob).ops]
    assert 15 in kinds, (wl.name, kinds)
    outs = [np.full(s, 0x55, dtype=dt) for s, dt in wl.outputs]
    desc_interp.run(blob, list(wl.inputs) + outs)
    prog.check_grouped_linear(wl, outs, _exact, prog.assert_bit_exact)


@pytest.mark.parametrize("seed", range(12))
def test_drawn_attention_records(seed):
    wl = w.attention_workload(**draw_attention(seed))
    blob = wl.program.serialize()
    outs = [np.full(s, 0x55, dtype=dt) for s, dt in wl.outputs]
    desc_interp.run(blob, list(wl.inputs) + outs)
    prog.check_attention(wl, outs, _exact)


@pytest.fixture(scope="module")
def device():
    dev = thip.Device(0)
    yield dev
    dev.close()


def _run_gpu(device, wl):
    exe = thip.Executable(device, wl.program.serialize())
    outs = [np.full(s, 0x55, dtype=dt) for s, dt in wl.outputs]
    ptrs = [device.upload(a) for a in wl.inputs] + [device.upload(o) for o in outs]
    lens = [a.nbytes for a in wl.inputs] + [o.nbytes for o in outs]
    try:
        exe.run_device(ptrs, lens)
        n = len(wl.inputs)
        return [device.download(ptrs[n + i], o.shape, o.dtype) for i, o in enumerate(outs)], exe.op_kernels()
    finally:
        exe.close()
        for q in ptrs:
            device.free(q)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(64))
def test_gpu_drawn_grouped_linear(device, seed):
    case = draw_linear(seed)
    print("grouped linear", case, flush=True)
    wl = w.grouped_linear_workload(**case)
    outs, kernels = _run_gpu(device, wl)
    # one record, or (a pair whose two matrices do not fit a CU's LDS together) the two linears in one and the add behind it
    assert kernels[0].startswith("dec_linear<") and all(k.startswith("add_bf16<") for k in kernels[1:]) and len(kernels) <= 2, kernels
    prog.check_grouped_linear(wl, outs, prog.assert_bf16_close, prog.assert_bit_exact)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(24))
def test_gpu_drawn_attention(device, seed):
    case = draw_attention(seed)
    print("attention", case, flush=True)
    wl = w.attention_workload(**case)
    outs, kernels = _run_gpu(device, wl)
    assert all(k.startswith(("dec_matmul<", "fc_bf16", "transpose")) for k in kernels), kernels
    prog.check_attention(wl, outs, prog.assert_bf16_close)
