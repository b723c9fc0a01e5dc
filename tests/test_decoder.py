"""Decode-shaped bf16 programs: views, the grouped linear records, the transposed matmul operand read in place, and
the decoder step of benchmark configuration 4 (linears on block-quantized int8 weights, attention matmuls on the
caches, residual adds, the vocabulary projection) -- each op checked on the inputs the run gave it, at <= 1 bf16 ULP
(the adds bit-exactly), through the C-ABI on the GPU and through the descriptor interpreter on the CPU."""
import collections

import numpy as np
import pytest

import desc_interp
import torq_compiler_amd as thip
from oracle import programs as prog
from torq_compiler_amd import workloads as w

SMALL = dict(layers=2, hidden=256, heads=2, head_dim=64, ffn=384, vocab=512, cache_len=64, block=128)
K_DEC_LINEAR, K_DEC_MATMUL, K_FC_BF16, K_TRANSPOSE, K_ADD_BF16 = 15, 16, 8, 1, 9


def _case_id(case):
    return "-".join(str(v).replace(" ", "") for v in case.values())


def _kinds(blob):
    return [int(o["kind"]) for o in desc_interp.Descriptor(blob).ops]


def _interp(wl):
    blob = wl.program.serialize()
    outs = [np.full(s, 0x55, dtype=dt) for s, dt in wl.outputs]
    desc_interp.run(blob, list(wl.inputs) + outs)
    return blob, outs


# ---- CPU: the emitter's records through the descriptor interpreter ----------------------------------------------

@pytest.mark.parametrize("batch", [1, 3, 17])
@pytest.mark.parametrize("expose", [True, False])
def test_decoder_step_records(batch, expose):
    wl = w.decoder_step_workload(batch=batch, expose=expose, **SMALL)
    blob, outs = _interp(wl)
    # per layer: q/k/v in one record, the two attention matmuls reading the caches in place (no transpose records),
    # o + add, gate / up + add, down + add; then the vocabulary projection
    assert _kinds(blob) == [K_DEC_LINEAR, K_DEC_MATMUL, K_DEC_MATMUL, K_DEC_LINEAR, K_DEC_LINEAR, K_DEC_LINEAR] * SMALL["layers"] + [K_DEC_LINEAR]
    if expose:
        prog.check_decoder_step(wl, outs, prog.assert_bf16_close, prog.assert_bit_exact)
    ref = prog.eval_decoder_step(wl)
    # the interpreter evaluates every record with the oracle's functions: the whole chain then agrees bit for bit
    assert np.array_equal(outs[0][:, ref["columns"]], ref["logits"]) and np.array_equal(outs[1], ref["k"]) and np.array_equal(outs[2], ref["v"])


def test_decoder_step_without_fusion(monkeypatch):
    monkeypatch.setenv("THIP_NO_DECODE_FUSION", "1")
    wl = w.decoder_step_workload(batch=2, expose=True, **SMALL)
    blob, outs = _interp(wl)
    kinds = collections.Counter(_kinds(blob))
    assert K_DEC_LINEAR not in kinds and K_DEC_MATMUL not in kinds
    # seven linears per layer, and the attention matmuls as one record per sequence
    assert kinds[K_FC_BF16] == (7 + 2 * 2) * SMALL["layers"] + 1 and kinds[K_ADD_BF16] == 3 * SMALL["layers"]
    prog.check_decoder_step(wl, outs, prog.assert_bf16_close, prog.assert_bit_exact)


GROUPED = [dict(mode="single"), dict(mode="concat"), dict(mode="pair"), dict(mode="pair_hidden"), dict(mode="residual", K=256, N=256),
           dict(mode="residual_first", K=128, N=128), dict(mode="single", zero_points=True), dict(mode="pair", zero_points=True, expand_clamp=(-0.01, 0.02)),
           dict(mode="concat", clamp=(-0.5, 0.75), M=32), dict(mode="single", K=1152, N=48, block=1152, M=9), dict(mode="residual", K=384, N=384, block=384, M=1)]


@pytest.mark.parametrize("case", GROUPED, ids=_case_id)
def test_grouped_linear_records(case):
    wl = w.grouped_linear_workload(**case)
    blob, outs = _interp(wl)
    assert _kinds(blob) == [K_DEC_LINEAR]
    prog.check_grouped_linear(wl, outs, prog.assert_bf16_close, prog.assert_bit_exact)


@pytest.mark.parametrize("case", [dict(K=192), dict(block=64), dict(M=33), dict(N=24)], ids=_case_id)
def test_shapes_the_grouped_kernel_does_not_take(case):
    # K no multiple of 128, quantisation blocks below 128, more than 32 rows, N no multiple of 16: the general kernels run them
    args = dict(M=3, K=256, N=64, mode="concat", block=128)
    args.update(case)
    if "K" in case:
        args["block"] = 64
    wl = w.grouped_linear_workload(**args)
    blob, outs = _interp(wl)
    assert K_DEC_LINEAR not in _kinds(blob)
    prog.check_grouped_linear(wl, outs, prog.assert_bf16_close, prog.assert_bit_exact)


def test_views():
    p = thip.Program()
    b = p.binding(0, (4, 6, 8), np.uint16)
    v = p.view(b, (2, 24), offset=48)
    vv = p.view(v, (3, 8), offset=24)  # a view of a view names the binding: elements 72 .. 95
    with pytest.raises(thip.ThipError) as e:
        p.view(b, (4, 6, 9))
    assert e.value.code == thip.runtime.INVALID_ARGUMENT and "outside" in str(e.value)
    with pytest.raises(thip.ThipError):
        p.view(v, (2, 24), offset=1)
    with pytest.raises(thip.ThipError) as e:
        p.view(p.constant(np.zeros((2, 2), np.int8)), (4,))
    assert e.value.code == thip.runtime.UNIMPLEMENTED
    # out[3, 8] = (elements 72 .. 95 of the binding) + (elements 0 .. 23)
    out = p.binding(1, (3, 8), np.uint16)
    p.add(vv, p.view(b, (3, 8)), w.to_bf16(np.array([1.0, 1.0], np.float32)), np.zeros(1, np.float32), init=out, output_zp=0,
          output_min=w.NO_CLAMP[0], output_max=w.NO_CLAMP[1], shift_factor=0)
    x = w.to_bf16(np.arange(192, dtype=np.float32).reshape(4, 6, 8))
    res = np.zeros((3, 8), np.uint16)
    desc_interp.run(p.serialize(), [x, res])
    assert np.array_equal(w.from_bf16_np(res).reshape(-1), np.arange(72, 96) + np.arange(24))


def test_transposed_operand_is_read_in_place():
    # matmul(a, transpose(b)) with b a run-time [B, N, K] tensor: one record, no transpose; with more than 32 rows the general path
    for M, fused in ((4, True), (40, False)):
        rng = np.random.default_rng(5)
        a = w.to_bf16(rng.standard_normal((3, M, 64)))
        b = w.to_bf16(rng.standard_normal((3, 48, 64)))
        p = thip.Program()
        out = p.binding(2, (3, M, 48), np.uint16)
        bt = p.transpose(p.binding(1, b.shape, np.uint16), (0, 2, 1))
        p.matmul(p.binding(0, a.shape, np.uint16), bt, np.array([0.25], np.float32), init=out, output_zp=0, output_min=w.NO_CLAMP[0],
                 output_max=w.NO_CLAMP[1], shift=0)
        blob = p.serialize()
        assert (_kinds(blob) == [K_DEC_MATMUL]) == fused
        res = np.zeros((3, M, 48), np.uint16)
        desc_interp.run(blob, [a, b, res])
        want = prog.orc.matmul_bf16(a, np.ascontiguousarray(b.transpose(0, 2, 1)), np.array([0.25], np.float32))
        assert np.array_equal(res, want)


ATTENTION = [dict(B=1, H=4, D=256, T=1024, D2=256), dict(B=3, H=1, D=32, T=64, D2=16), dict(B=2, H=16, D=64, T=128, D2=48),
             dict(B=5, H=7, D=96, T=192, D2=80, bias=(0.5, -0.25), clamp1=(-1.0, 1.5), clamp2=(-0.5, 0.75)),
             dict(B=1, H=4, D=128, T=256, D2=64, rank2=True)]


@pytest.mark.parametrize("case", ATTENTION + [dict(B=2, H=4, D=64, T=96, D2=24)], ids=_case_id)
def test_attention_records(case):
    """scores = q K^T, context = scores V with the scores an intermediate: two records reading the caches in place."""
    wl = w.attention_workload(**case)
    blob, outs = _interp(wl)
    assert _kinds(blob) == [K_DEC_MATMUL, K_DEC_MATMUL]
    prog.check_attention(wl, outs, lambda g, want, what, magnitude=None: prog.assert_bit_exact(g, want, what))


# ---- GPU ----------------------------------------------------------------------------------------------------------

def _run_gpu(device, wl, dispatches=1):
    exe = thip.Executable(device, wl.program.serialize())
    outs = [np.full(s, 0x55, dtype=dt) for s, dt in wl.outputs]
    ptrs = [device.upload(a) for a in wl.inputs] + [device.upload(o) for o in outs]
    lens = [a.nbytes for a in wl.inputs] + [o.nbytes for o in outs]
    try:
        results = []
        for _ in range(dispatches):  # the first dispatch runs eagerly, the second is captured, later ones replay the graph
            exe.run_device(ptrs, lens)
            n = len(wl.inputs)
            results.append([device.download(ptrs[n + i], o.shape, o.dtype) for i, o in enumerate(outs)])
        return results, exe.op_kernels()
    finally:
        exe.close()
        for q in ptrs:
            device.free(q)


@pytest.fixture(scope="module")
def device():
    dev = thip.Device(0)
    yield dev
    dev.close()


@pytest.mark.gpu
@pytest.mark.parametrize("batch", [1, 32])
def test_gpu_decoder_step_full_width(device, batch):
    """Two layers at the benchmark's widths and the FULL 1152 -> 262144 vocabulary projection (sampled columns)."""
    wl = w.decoder_step_workload(batch=batch, layers=2, expose=True)
    results, kernels = _run_gpu(device, wl, dispatches=3)
    fam = collections.Counter(k.split("<")[0] for k in kernels)
    assert fam == {"dec_linear": 8, "dec_matmul": 4, "fc_bf16_wide": 1}, fam
    for outs in results:
        prog.check_decoder_step(wl, outs, prog.assert_bf16_close, prog.assert_bit_exact)
    for outs in results[1:]:  # eager, captured and replayed dispatches agree bit for bit
        assert all(np.array_equal(a, b) for a, b in zip(outs, results[0]))


@pytest.mark.gpu
@pytest.mark.parametrize("batch", [2, 4, 5, 16, 17])
def test_gpu_decoder_step_batches(device, batch):
    # 2 and 4 rows: the input rows come through LDS; 5 and 16: through registers, one row group; 17: two row groups
    wl = w.decoder_step_workload(batch=batch, layers=2, vocab=4096, expose=True)
    results, kernels = _run_gpu(device, wl)
    prog.check_decoder_step(wl, results[0], prog.assert_bf16_close, prog.assert_bit_exact)
    linears = [k for k in kernels if k.startswith("dec_linear")]
    if batch <= 4:
        # the down projection's four rows of 6912 no longer fit LDS next to its weights: it alone takes the register path
        through_lds = [k.startswith("dec_linear<1,1,1,") for k in linears]
        assert all(through_lds) if batch <= 2 else (sum(through_lds) == len(linears) - 2 and all(k.startswith(("dec_linear<1,1,1,", "dec_linear<1,2,0,")) for k in linears)), kernels
    else:
        # (few column tiles share their rows out over several workgroups, each with at most 16 of them)
        assert all(k.startswith(("dec_linear<1,2,0,", "dec_linear<2,1,0,") if batch > 16 else "dec_linear<1,2,0,") for k in linears), kernels


@pytest.mark.gpu
def test_gpu_decoder_step_hidden_intermediates(device):
    """The program as the benchmark times it (intermediates not exposed): keys, values and logits against the oracle's
    own run of the chain.  A bf16 rounding that differs once is carried through every later op, so the whole chain is
    compared in the large: the keys and values of layer 0 (one op deep) at one ULP, the logits by their mean error."""
    wl = w.decoder_step_workload(batch=2, layers=3, vocab=8192)
    results, _ = _run_gpu(device, wl)
    logits, knew, vnew = results[0]
    ref = prog.eval_decoder_step(wl)
    prog.assert_bf16_close(knew[0], ref["k"][0], "keys of layer 0")
    prog.assert_bf16_close(vnew[0], ref["v"][0], "values of layer 0")
    got = prog.orc.from_bf16(logits[:, ref["columns"]]).astype(np.float64)
    want = prog.orc.from_bf16(ref["logits"]).astype(np.float64)
    assert np.sqrt(np.mean((got - want) ** 2)) < 0.01 * np.sqrt(np.mean(want ** 2))


@pytest.mark.gpu
@pytest.mark.parametrize("case", GROUPED + [dict(mode="pair", K=1152, N=6912, M=1), dict(mode="residual", K=1024, N=1024, M=32),
                                           dict(mode="single", K=6912, N=1152, M=4), dict(mode="single", K=6912, N=1152, M=20)],
                         ids=_case_id)
def test_gpu_grouped_linear(device, case):
    wl = w.grouped_linear_workload(**case)
    results, kernels = _run_gpu(device, wl)
    assert len(kernels) == 1 and kernels[0].startswith("dec_linear<"), kernels
    prog.check_grouped_linear(wl, results[0], prog.assert_bf16_close, prog.assert_bit_exact)


@pytest.mark.gpu
@pytest.mark.parametrize("case", ATTENTION + [dict(B=32, H=4, D=256, T=1024, D2=256), dict(B=2, H=4, D=256, T=4096, D2=256)], ids=_case_id)
def test_gpu_attention(device, case):
    """One decode step of attention with the scores hidden between its two matmuls, against the oracle's two matmuls;
    eager, captured and replayed dispatches agree bit for bit."""
    wl = w.attention_workload(**case)
    results, kernels = _run_gpu(device, wl, dispatches=3)
    assert [k.split("<")[0] for k in kernels] == ["dec_matmul", "dec_matmul"], kernels
    for outs in results:
        prog.check_attention(wl, outs, prog.assert_bf16_close)
    assert all(np.array_equal(outs[0], results[0][0]) for outs in results[1:])


@pytest.mark.gpu
def test_gpu_transposed_operand_read_in_place(device):
    rng = np.random.default_rng(6)
    for B, M, K, N in ((3, 4, 256, 1024), (2, 4, 1024, 256), (1, 20, 264, 50), (5, 1, 8, 3)):
        a = w.to_bf16(rng.standard_normal((B, M, K)))
        b = w.to_bf16(rng.standard_normal((B, N, K)) / np.sqrt(K))
        p = thip.Program()
        out = p.binding(2, (B, M, N), np.uint16)
        bt = p.transpose(p.binding(1, b.shape, np.uint16), (0, 2, 1))
        p.matmul(p.binding(0, a.shape, np.uint16), bt, np.array([0.25], np.float32), init=out, output_zp=0, output_min=w.NO_CLAMP[0],
                 output_max=w.NO_CLAMP[1], shift=0)
        wl = w.Workload("matmulT_%dx%dx%dx%d" % (B, M, K, N), p, [a, b], [((B, M, N), np.uint16)], 0, 0)
        results, kernels = _run_gpu(device, wl)
        assert len(kernels) == 1 and kernels[0].startswith("dec_matmul<"), kernels
        bT = np.ascontiguousarray(b.transpose(0, 2, 1))
        want = prog.orc.matmul_bf16(a, bT, np.array([0.25], np.float32))
        mag = np.einsum("bmk,bkn->bmn", np.abs(prog.orc.from_bf16(a).astype(np.float64)), np.abs(prog.orc.from_bf16(bT).astype(np.float64))) + 0.25
        prog.assert_bf16_close(results[0][0], want, wl.name, magnitude=mag)
