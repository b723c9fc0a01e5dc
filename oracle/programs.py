"""Whole workloads evaluated with the CPU oracle, and the comparisons the checkers use.

Test infrastructure: the product never imports this module.  A workload (torq_compiler_amd.workloads.Workload)
carries its ops' parameters in ``attrs``; these functions replay them with the oracle's functions:
``eval_workload`` for a single-op workload, ``eval_network`` for a layer list, ``check_decoder_step`` /
``eval_decoder_step`` for the decoder-step program.
"""
import numpy as np

from . import oracle as orc


def eval_workload(wl):
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
    if kind == "fcbf16":
        return [orc.fully_connected_bf16(x, a["weights"], a["bias"], output_min=a["output_min"], output_max=a["output_max"])]
    if kind in ("convbf16", "dwbf16"):
        fn = orc.conv2d_bf16 if kind == "convbf16" else orc.depthwise_conv2d_bf16
        return [fn(x, a["weights"], a["bias"], pad=a["pad"], stride=a["stride"], output_min=a["output_min"], output_max=a["output_max"],
                   layout=orc.NHWC if a["nhwc"] else orc.NCHW)]
    if kind == "pwadd":
        wp, sbp, pa = a["pw"]
        aw, asb, aa = a["add"]
        y = orc.conv2d(x, wp, sbp, layout=orc.NHWC, **pa)
        return [orc.add(wl.inputs[1], y, aw, asb, **aa) if a["other_first"] else orc.add(y, wl.inputs[1], aw, asb, **aa)]
    if kind == "branches":
        ya, yb, yc = [orc.fully_connected(x, wt, sb, **at) for wt, sb, at in a["fcs"]]
        (w0, sb0, a0), (w1, sb1, a1) = a["adds"]
        return [orc.add(orc.add(ya, yb, w0, sb0, **a0), yc, w1, sb1, **a1)]
    if kind == "fma":
        return [orc.fma(x, a.pop("weights"), a.pop("scale_bias"), **a)]
    if kind == "mul":
        return [orc.mul(x, wl.inputs[1], a.pop("scale_bias"), **a)]
    if kind == "binary":
        return [orc.elementwise_binary(a["op_type"], x, wl.inputs[1], is_unsigned=a["is_unsigned"])]
    if kind == "compare":
        return [orc.elementwise_compare(a["op_type"], x, wl.inputs[1], is_unsigned=a["is_unsigned"])]
    if kind == "unary":
        return [orc.elementwise_unary(a["op_type"], x)]
    if kind == "shift":
        return [orc.elementwise_shift(a["op_type"], x, wl.inputs[1], round=a["round"])]
    if kind == "table":
        return [orc.table(x, a["words"], a["out_dtype"])]
    if kind == "act":
        return [orc.act(x, a["name"], min_int=a["min_int"], max_int=a["max_int"], out_dtype=a["out_dtype"])]
    if kind == "avgpoolbf16":
        return [orc.avg_pool2d_bf16(x, a["weights"], a["bias"], output_min=a["output_min"], output_max=a["output_max"])]
    if kind == "expandmm":
        w16 = orc.expand_weights(a["weights"], a["scale"], a["qbias"], block_size=a["block"], output_min=a["expand_min"],
                                 output_max=a["expand_max"])
        res = [orc.matmul_bf16(x, w16, a["bias"], output_min=a["output_min"], output_max=a["output_max"])]
        return res if a["fold"] else res + [w16[None]]
    if kind == "addbf16":
        return [orc.add_bf16(wl.inputs[0], wl.inputs[1], a["weights"], a["bias"], output_min=a["output_min"], output_max=a["output_max"])]
    if kind == "matmul":
        res = orc.matmul(x, a["input2"], a["scale_bias"], output_zp=a["output_zp"], output_min=a["output_min"], output_max=a["output_max"],
                         shift=a["shift"], out_dtype=a["out_dtype"])
        return [res.reshape(wl.outputs[0][0])]
    if kind == "matmulbf16":
        res = orc.matmul_bf16(x, a["input2"], a["bias"])
        return [res.reshape(wl.outputs[0][0])]
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


def assert_bit_exact(got, want, what=""):
    assert got.shape == want.shape and got.dtype == want.dtype, (what, got.shape, want.shape, got.dtype, want.dtype)
    if not np.array_equal(got, want):
        bad = np.argwhere(got != want)
        first = tuple(bad[0])
        raise AssertionError("%s: %d of %d elements differ; first at %s: got %d want %d"
                             % (what, len(bad), got.size, first, int(got[first]), int(want[first])))


def bf16_ordered(bits):
    """bf16 bit patterns -> integers whose order and spacing are those of the values (one step = one ULP)."""
    b = np.asarray(bits, dtype=np.uint16).astype(np.int32)
    return np.where(b < 0x8000, b, 0x8000 - b)


# Tally of the bf16 comparisons of this process: per call, (what, elements compared, elements beyond `ulps` steps that
# only the cancellation bound admitted).  tests/test_bf16.py reports and bounds it after its GPU cases.
BF16_TALLY = []


def assert_bf16_close(got, want, what="", ulps=1, magnitude=None):
    """The bf16 rows are tolerance rows: at most `ulps` bf16 steps from the oracle per element.

    `magnitude` (sum of |products| + |bias| per element) admits, for sums that cancel, the error a different
    order of fp32 additions can make: 2^-17 of it (a bf16 step is 2^-8 of the result, so where nothing cancels the
    ULP bound is the binding one)."""
    assert got.shape == want.shape and got.dtype == np.uint16 and want.dtype == np.uint16, (what, got.shape, want.shape)
    bad = np.abs(bf16_ordered(got) - bf16_ordered(want)) > ulps
    if magnitude is not None:
        gf = (got.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        wf = (want.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        beyond = int(bad.sum())
        bad &= ~(np.abs(gf - wf) <= np.asarray(magnitude, dtype=np.float64).reshape(got.shape) * 2.0 ** -17)
        BF16_TALLY.append((what, int(got.size), beyond - int(bad.sum())))
    else:
        BF16_TALLY.append((what, int(got.size), 0))
    if bad.any():
        first = tuple(np.argwhere(bad)[0])
        raise AssertionError("%s: %d of %d elements differ by more than %d bf16 ULP; first at %s: got 0x%04x want 0x%04x"
                             % (what, int(bad.sum()), got.size, ulps, first, int(got[first]), int(want[first])))


def eval_network(wl, return_all=False):
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


# ---- decoder step (benchmark configuration 4) ----------------------------------------------------------------

def _f64(bits):
    return orc.from_bf16(bits).astype(np.float64)


def _decoder_op(op, src, caches, batch, rows, columns=None):
    """One op of a decoder-step workload on the given bf16 inputs, for the batch rows `rows` (indices into the
    `batch` sequences of the workload; src holds those rows only): (result, magnitude).  magnitude = sum of
    |products| + |bias| per element, what the cancellation allowance of assert_bf16_close is measured against.
    columns: for a linear, the output columns to compute (the vocabulary projection is checked on a sample)."""
    pr = op.params
    R = len(rows)
    if op.kind == "linear":
        wq, scale, qbias = pr["weights"], pr["scale"], pr["qbias"]
        if columns is not None:
            wq, scale, qbias = wq[:, columns], scale[:, columns], qbias[:, columns]
        w16 = orc.expand_weights(np.ascontiguousarray(wq), np.ascontiguousarray(scale), np.ascontiguousarray(qbias), block_size=pr["block"],
                                 output_min=pr.get("expand_min", orc.NO_CLAMP_MIN), output_max=pr.get("expand_max", orc.NO_CLAMP_MAX))
        x = src[0].reshape(R, wq.shape[0])
        # input2 of the matmul is the K x N expansion; summed over k in order like every oracle matmul
        want = orc.matmul_bf16(x, w16, np.zeros(1, np.float32), output_min=pr.get("output_min", orc.NO_CLAMP_MIN),
                               output_max=pr.get("output_max", orc.NO_CLAMP_MAX))[0]
        return want, np.abs(_f64(x)) @ np.abs(_f64(w16))
    if op.kind in ("scores", "context"):
        kc, vc = caches
        heads = op.shape[1]
        a = src[0].reshape(R, heads, -1)
        sel = [pr["layer"] * batch + r for r in rows]
        cache = kc[sel] if op.kind == "scores" else vc[sel]
        rhs = np.ascontiguousarray(cache.transpose(0, 2, 1))  # what the torq_hl.transpose in front of the matmul delivers
        want = orc.matmul_bf16(a, rhs, np.zeros(1, np.float32))
        return want, np.einsum("bmk,bkn->bmn", np.abs(_f64(a)), np.abs(_f64(rhs)))
    if op.kind == "add":
        shape = (R,) + op.shape[1:]
        return orc.add_bf16(src[0].reshape(shape), src[1].reshape(shape), pr["weights"], pr["bias"]), None
    raise ValueError(op.kind)


def vocabulary_sample(vocab, count=2048, seed=7):
    """Columns of the vocabulary projection that the checkers compute: the first and last 64 and a seeded sample."""
    if vocab <= count:
        return np.arange(vocab)
    rng = np.random.default_rng(seed)
    cols = np.concatenate([np.arange(64), np.arange(vocab - 64, vocab), rng.choice(vocab, size=count - 128, replace=False)])
    return np.unique(cols)


def check_decoder_step(wl, outputs, compare_close, compare_exact, rows=None):
    """Every op of an exposed decoder-step workload (expose=True) checked on the inputs the GPU gave it: the
    oracle evaluates the op on the GPU's own intermediates, so one op's rounding does not reach the next comparison.
    outputs: the program's output arrays (logits, new keys, new values, trace).  compare_close(got, want, what,
    magnitude) for the matmuls (tolerance rows), compare_exact(got, want, what) for the adds.  rows: the sequences
    to check (all when None; a sequence's step depends on its own row and caches only)."""
    a = wl.attrs
    assert a["expose"], "needs the workload built with expose=True"
    logits, knew, vnew, trace = outputs
    x_in, kc, vc = wl.inputs
    M = a["batch"]
    rows = list(range(M)) if rows is None else list(rows)
    tensors = {"x_in": x_in[rows]}
    for name, (off, shape) in a["trace"].items():
        tensors[name] = trace[off:off + int(np.prod(shape))].reshape(shape)[rows]
    for l in range(a["layers"]):
        tensors["k%d" % l] = knew[l][rows]
        tensors["v%d" % l] = vnew[l][rows]
    cols = vocabulary_sample(a["vocab"])
    tensors["logits"] = logits[rows][:, cols]
    for op in wl.attrs["ops"]:
        src = [tensors[n] for n in op.inputs]
        want, mag = _decoder_op(op, src, (kc, vc), M, rows, columns=cols if op.out == "logits" else None)
        got = tensors[op.out]
        if op.kind == "add":
            compare_exact(got.reshape(want.shape), want, "%s %s" % (wl.name, op.out))
        else:
            compare_close(got.reshape(want.shape), want, "%s %s" % (wl.name, op.out), magnitude=mag.reshape(want.shape))


def eval_decoder_step(wl, rows=None):
    """The oracle's own run of the whole chain for the given batch rows (all when None): every op on the oracle's
    previous results.  Returns {"logits": sampled columns, "columns": their indices, "k": [layers, rows, d],
    "v": likewise}.  A sequence's step depends on its own row and caches only, so a subset of rows is exact."""
    a = wl.attrs
    x_in, kc, vc = wl.inputs
    rows = list(range(a["batch"])) if rows is None else list(rows)
    tensors = {"x_in": x_in[rows]}
    cols = vocabulary_sample(a["vocab"])
    for op in wl.attrs["ops"]:
        src = [tensors[n] for n in op.inputs]
        want, _ = _decoder_op(op, src, (kc, vc), a["batch"], rows, columns=cols if op.out == "logits" else None)
        tensors[op.out] = want
    L = a["layers"]
    return dict(logits=tensors["logits"], columns=cols, k=np.stack([tensors["k%d" % l] for l in range(L)]),
                v=np.stack([tensors["v%d" % l] for l in range(L)]))


def _bf16_step(bits):
    """The distance from each bf16 value to the next one up in magnitude."""
    return np.spacing(np.abs(orc.from_bf16(np.asarray(bits, dtype=np.uint16))).astype(np.float32)).astype(np.float64) * 65536.0


def check_grouped_linear(wl, outputs, compare_close, compare_exact):
    """A grouped_linear_workload's outputs, each op on the inputs the GPU gave it (hidden intermediates of a
    "pair_hidden" program are the oracle's own: what the add reads is then one rounding further from a binding)."""
    tensors = {"x_in": wl.inputs[0]}
    for name, arr in zip(wl.attrs["names"], outputs):
        tensors[name] = arr
    M = wl.inputs[0].shape[0]
    rows = list(range(M))
    for op in wl.attrs["ops"]:
        src = [tensors[n] for n in op.inputs]
        want, mag = _decoder_op(op, src, None, M, rows)
        if op.out not in tensors:
            tensors[op.out] = want  # never stored by the program
            continue
        got = tensors[op.out]
        hidden_inputs = any(n not in wl.attrs["names"] and n != "x_in" for n in op.inputs)
        if op.kind == "add" and not hidden_inputs:
            compare_exact(got.reshape(want.shape), want, "%s %s" % (wl.name, op.out))
        elif op.kind == "add":
            # each hidden operand may be one bf16 step from the oracle's: the sum moves by at most the weighted steps
            # of both, plus one step of its own rounding
            w0, w1 = (abs(float(v)) for v in orc.from_bf16(op.params["weights"])[:2])
            room = w0 * _bf16_step(src[0]) + w1 * _bf16_step(src[1]) + _bf16_step(want)
            bad = np.abs(_f64(got.reshape(want.shape)) - _f64(want)) > room.reshape(want.shape)
            assert not bad.any(), "%s %s: %d elements beyond the propagated bound" % (wl.name, op.out, int(bad.sum()))
        else:
            compare_close(got.reshape(want.shape), want, "%s %s" % (wl.name, op.out), magnitude=mag.reshape(want.shape))


def check_attention(wl, outputs, compare_close):
    """An attention_workload's context against the two matmuls it stands for (orc.matmul_bf16 twice, the scores
    rounded to bf16 in between).  The scores never leave the GPU, so the context is checked on the oracle's scores,
    with room for the one thing that may differ: a score whose exact value lies within 2^-20 of its sum of |products| of a bf16
    rounding boundary (some twenty standard deviations of what the order of fp32 additions moves a sum of this kind
    by; about one score in a hundred) may be either neighbour, and moves the
    context by its bf16 step times the value it multiplies (plus, for the contexts it moves, one step of their own
    rounding)."""
    q, keys, vals = wl.inputs
    if q.ndim == 2:
        q, keys, vals = q[None], keys[None], vals[None]
    b1 = np.array([wl.attrs["bias"][0]], np.float32)
    b2 = np.array([wl.attrs["bias"][1]], np.float32)
    lo1, hi1 = wl.attrs["clamp1"]
    lo2, hi2 = wl.attrs["clamp2"]
    kT = np.ascontiguousarray(keys.transpose(0, 2, 1))
    vT = np.ascontiguousarray(vals.transpose(0, 2, 1))
    scores = orc.matmul_bf16(q, kT, b1, output_min=lo1, output_max=hi1)
    want = orc.matmul_bf16(scores, vT, b2, output_min=lo2, output_max=hi2)
    exact = np.einsum("bhd,bdt->bht", _f64(q), _f64(kT)) + float(b1[0])
    mag1 = np.einsum("bhd,bdt->bht", np.abs(_f64(q)), np.abs(_f64(kT))) + abs(float(b1[0]))
    sf = _f64(scores)
    step = _bf16_step(scores)
    boundary = sf + np.where(exact >= sf, 0.5, -0.5) * step
    either = np.abs(exact - boundary) <= mag1 * 2.0 ** -20
    room = np.einsum("bht,btd->bhd", either * step, np.abs(_f64(vT)))
    mag2 = np.einsum("bht,btd->bhd", np.abs(sf), np.abs(_f64(vT))) + abs(float(b2[0]))
    got = outputs[0].reshape(want.shape)
    # (a context moved by such a score is rounded again: one more step of its own)
    room = np.where(room > 0, room + _bf16_step(want), 0.0)
    compare_close(got, want, wl.name, magnitude=mag2 + room * 2.0 ** 17)
    return int(either.sum()), int(either.size)
