#!/usr/bin/env python3
"""Benchmark of the quantized TorqHL operator path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu] [--no-others]

A "step" is one dispatch of the workload's program (inputs resident in HBM).  Before the W warm-up steps of every
workload the card is kept busy with it for --precondition-ms (200 by default, untimed, reported in the JSON): an idle
card sits at its lowest clocks, and a few milliseconds of timed steps right after that measure the ramp.  The default workload
is the int8 fully_connected (4096, 4096, 4096) with fused per-column requant, the largest
single-GPU case of the benchmark's matmul configuration; its metric is int8 GOP/s (1 MAC = 2 ops)
against the dense int8 MFMA peak.  The other benchmark shapes are measured briefly in the same run
and reported under "per_op" with the roofline that bounds each.

The CPU leg (skipped with --no-cpu) times the CPU oracle on a bounded sample of the default workload
("cpu_baseline") and uses the same oracle to check this run's GPU results ("parity_checked"); nothing
else here touches it.

Prints ONE JSON line.
"""
import argparse
import hashlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0   # MI355X dense int8 MFMA, TOP/s
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E, GB/s
# bandwidth rows are timed on buffer sets that together exceed this many bytes (twice the 256 MiB last-level cache),
# dispatch i on set i mod n, so that every dispatch finds its operands in HBM
COLD_WORKING_SET = 512 << 20
MAX_BUFFER_SETS = 160


def import_package():
    import __graft_entry__ as entry
    return entry._import_package()


def workload_table(pkg):
    w = pkg.workloads
    return {
        "fc_4096x4096x4096": (lambda: w.fully_connected_workload(4096, 4096, 4096), "mfma"),
        "fc_512x4096x4096": (lambda: w.fully_connected_workload(512, 4096, 4096), "mfma"),
        "fc_16x2048x8192": (lambda: w.fully_connected_workload(16, 2048, 8192), "hbm"),
        "fc_1x2048x2048": (lambda: w.fully_connected_workload(1, 2048, 2048), "hbm"),
        "conv_112x112x32_o64_3x3": (lambda: w.conv2d_workload(), "mfma"),
        # large convolutions (the benchmark's own convolution is 0.46 GOP): 3x3 over 256 / 512 channels at batch 32, 118 GOP each,
        # and a pointwise expansion whose K is short
        "conv3x3_56x56x256_o256_b32": (lambda: w.conv2d_workload(N=32, H=56, W=56, C=256, O=256, realistic=True), "mfma"),
        "conv3x3_28x28x512_o512_b32": (lambda: w.conv2d_workload(N=32, H=28, W=28, C=512, O=512, realistic=True), "mfma"),
        # a channel count that is no multiple of the 64-byte k-tile: k-tiles straddle the window's taps
        "conv3x3_56x56x96_o96_b32": (lambda: w.conv2d_workload(N=32, H=56, W=56, C=96, O=96, realistic=True), "mfma"),
        # (26 MB in, 103 MB out, 53 GOP: 16 us of HBM traffic at 8 TB/s against 10.5 us of MFMA work at 5 POP/s -- the memory side bounds it)
        "conv1x1_56x56x256_o1024_b32": (lambda: w.conv2d_workload(N=32, H=56, W=56, C=256, O=1024, KH=1, KW=1, pad=(0, 0, 0, 0), realistic=True), "hbm"),
        "depthwise_b64": (lambda: w.depthwise_workload(N=64), "hbm"),
        "depthwise_b1": (lambda: w.depthwise_workload(N=1), "hbm"),
        "depthwise_s1_b256": (lambda: w.depthwise_workload(N=256, stride=(1, 1), pad=(1, 1, 1, 1)), "hbm"),
        "maxpool_b64": (lambda: w.maxpool_workload(N=64), "hbm"),
        "maxpool_b1": (lambda: w.maxpool_workload(N=1), "hbm"),
        "avgpool_b64": (lambda: w.avgpool_workload(N=64), "hbm"),
        "avgpool_b1": (lambda: w.avgpool_workload(N=1), "hbm"),
        "add_b64": (lambda: w.add_workload(N=64), "hbm"),
        "add_b1": (lambda: w.add_workload(N=1), "hbm"),
        # integer elementwise ops next to the convolution path, at the shape of the add row
        "rescale_b64": (lambda: w.fma_workload((64, 56, 56, 24)), "hbm"),
        "mul_b64": (lambda: w.mul_workload((64, 56, 56, 24)), "hbm"),
        # bf16 linears of a decoder layer (hidden 1152, MLP 6912) at 1 and 32 tokens: weight streaming
        "fcbf16_1x1152x6912": (lambda: w.fully_connected_bf16_workload(1, 1152, 6912), "hbm"),
        "fcbf16_32x1152x6912": (lambda: w.fully_connected_bf16_workload(32, 1152, 6912), "hbm"),
        "fcbf16_32x6912x1152": (lambda: w.fully_connected_bf16_workload(32, 6912, 1152), "hbm"),
        # a quarter of the vocabulary projection (1152 -> 262144) with bf16 weights, and with block-quantized int8
        # weights (torq_hl.expand_weights folded into the matmul: the int8 bytes are what is streamed)
        "fcbf16_1x1152x65536": (lambda: w.fully_connected_bf16_workload(1, 1152, 65536), "hbm"),
        "expandmm_1x1152x65536": (lambda: w.expand_weights_workload(M=1, K=1152, N=65536, block=128), "hbm"),
        "expandmm_32x1152x65536": (lambda: w.expand_weights_workload(M=32, K=1152, N=65536, block=128), "hbm"),
    }


def network_table(pkg):
    """Whole-network workloads (benchmark configurations 3 and 4); selectable with --workload."""
    w = pkg.workloads
    table = {"mbv2_b%d" % b: (lambda b=b: w.mobilenet_v2_workload(batch=b), "mfma") for b in (1, 32, 256)}
    table.update({"decoder_b%d" % b: (lambda b=b: w.decoder_step_workload(batch=b), "hbm") for b in DECODER_BATCHES})
    return table


DECODER_BATCHES = (1, 32)
# What a decode step is priced against: every int8 weight of the 26 layers and of the vocabulary projection once per
# step, whatever the batch (26 * 26 836 992 + 301 989 888 bytes).
DECODER_WEIGHT_BYTES = 999751680


def decoder_parity(pkg, dev, batch):
    """The decoder step checked against the oracle: a two-layer twin of the program at the same batch with every
    intermediate exposed, each op on the inputs the GPU gave it (<= 1 bf16 ULP, the adds bit-exact; every sequence at
    one token, the first and last otherwise), with the full-width vocabulary projection on sampled columns."""
    from oracle import programs as prog
    wl = pkg.workloads.decoder_step_workload(batch=batch, layers=2, expose=True)
    o = Loaded(pkg, dev, wl)
    try:
        o.exe.run_device(o.ptrs, o.lens)
        got = [o.output(i) for i in range(len(wl.outputs))]
        prog.check_decoder_step(wl, got, prog.assert_bf16_close, prog.assert_bit_exact, rows=None if batch <= 2 else [0, batch - 1])
        return True
    except AssertionError as e:
        print("decoder step differs from the oracle: %s" % e, file=sys.stderr)
        return False
    finally:
        o.close()


def decoder_row(pkg, dev, batch, pre_ms, check):
    """One decode step (26 layers + vocabulary projection) as ONE graph-replayed program: ms per step, steps and
    tokens per second, and the int8 weight bytes per second against HBM's 8 TB/s.  1 GB of weights per step: every
    step finds them cold.  The ops between these (normalisation, rotary embedding, softmax, the gate's activation)
    are not on this path, so the figure is for the linears and attention matmuls only."""
    o = Loaded(pkg, dev, pkg.workloads.decoder_step_workload(batch=batch))
    o.precondition(pre_ms)
    o.run(5)
    ms = min(o.run(20) for _ in range(3))
    names = o.exe.op_kernels()
    row = {"ms": round(ms, 4), "steps_per_s": round(1e3 / ms, 1), "tokens_per_s": round(batch * 1e3 / ms, 1), "kernels": len(names),
           "scope": "linears + attention matmuls + residual adds + vocabulary projection only", "weight_bytes": o.wl.attrs["weight_bytes"],
           "GB/s": round(o.wl.attrs["weight_bytes"] / (ms * 1e-3) / 1e9, 1), "frac": round(o.wl.attrs["weight_bytes"] / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 5),
           "kernel_families": sorted(set(k.split("<")[0] for k in names))}
    assert o.wl.attrs["weight_bytes"] == DECODER_WEIGHT_BYTES
    o.close()
    if check:
        row["parity_checked"] = decoder_parity(pkg, dev, batch)
    return row


class Loaded:
    """A workload resident on the GPU: executable + device buffers."""

    def __init__(self, pkg, dev, wl):
        self.wl = wl
        self.dev = dev
        self.exe = pkg.Executable(dev, wl.program.serialize())
        self.outs = [np.zeros(s, dtype=dt) for s, dt in wl.outputs]
        self.ptrs = [dev.upload(a) for a in wl.inputs] + [dev.upload(o) for o in self.outs]
        self.lens = [a.nbytes for a in wl.inputs] + [o.nbytes for o in self.outs]

    def run(self, iterations):
        """Returns mean ms per dispatch from HIP events on the executable's stream."""
        return self.exe.time_device(self.ptrs, self.lens, iterations)

    def precondition(self, milliseconds, dispatch=None):
        """Keeps the card busy with this workload for `milliseconds` of wall time, untimed: an idle card sits at its
        lowest clocks and takes some 100 ms of work to reach the ones it sustains, and a measurement of a few
        milliseconds taken before that reads 10-20 % slow."""
        dispatch = dispatch or self.run
        n, t0 = 20, time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < milliseconds:
            ms = dispatch(n)
            n = int(min(200, max(20, 2.0 / max(ms, 1e-4))))  # about 2 ms of work between synchronisations, a short queue

    def run_cold(self, iterations, precondition_ms=0.0, repeats=1):
        """The same on rotating copies of every binding (see COLD_WORKING_SET); returns (ms per dispatch, sets).  The best
        of `repeats` timed passes: the per-op rows are a millisecond of dispatches each, which one hiccup of the host doubles."""
        per_set = sum(self.lens)
        sets = int(min(MAX_BUFFER_SETS, max(2, -(-COLD_WORKING_SET // per_set))))
        hosts = list(self.wl.inputs) + self.outs
        extra = [[self.dev.upload(h) for h in hosts] for _ in range(sets - 1)]
        try:
            all_sets = [self.ptrs] + extra
            self.exe.time_device_rotating(all_sets, self.lens, sets)  # every set once: first touch
            self.precondition(precondition_ms, lambda n: self.exe.time_device_rotating(all_sets, self.lens, n))
            ms = min(self.exe.time_device_rotating(all_sets, self.lens, max(iterations, 2 * sets)) for _ in range(max(1, repeats)))
        finally:
            for ptrs in extra:
                for p in ptrs:
                    self.dev.free(p)
        return ms, sets

    def output(self, i=0):
        o = self.outs[i]
        return self.dev.download(self.ptrs[len(self.wl.inputs) + i], o.shape, o.dtype)

    def close(self):
        self.exe.close()
        for p in self.ptrs:
            self.dev.free(p)


# HBM bytes per launch of each workload's kernel, from rocprofv3 counters: FETCH_SIZE * 1.9995 + WRITE_SIZE * 1.0
# (KiB per dispatch; the factors are what the same counters read for a plain 256 MiB copy, --copy-calibration).
# They belong to the kernels as they were when the counters were read: TRAFFIC_SOURCES_SHA256 holds the hashes of
# the kernel sources (under torq-compiler_amd/csrc) at that time, and a run whose kernel source -- the file the
# workload's kernel lives in, or the helpers every kernel file includes -- has changed since reports traffic null.
TRAFFIC_SOURCES_SHA256 = {
    "thip_kernels_common.h": "9e7783387939bacca5e8a40e8a9859135213407975bcc967c50e4c8025feb72a",
    "thip_igemm.hip": "f2244679f589b21aad8bad523ae60b45d6b6f0838057052313d119ff49bbd712",
    "thip_bandwidth.hip": "f152f95926c1fabe7debb7b708689096163480bbd0983aff0dff443ebb6f1667",
}
MEASURED_TRAFFIC = {
    "fc_4096x4096x4096": (49385.0 * 1.9995 + 16581.2 * 1.0000) * 1024,
    "fc_512x4096x4096": (16453.0 * 1.9995 + 2048.0 * 1.0000) * 1024,
    "fc_16x2048x8192": (8408.0 * 1.9995 + 256.0 * 1.0000) * 1024,
    "conv_112x112x32_o64_3x3": (370.7 * 1.9995 + 784.0 * 1.0000) * 1024,
    "conv3x3_56x56x256_o256_b32": (17259.9 * 1.9995 + 25990.4 * 1.0000) * 1024,
    "conv1x1_56x56x256_o1024_b32": (14417.5 * 1.9995 + 100352.0 * 1.0000) * 1024,
    "depthwise_b64": (14212.7 * 1.9995 + 7810.1 * 1.0000) * 1024,
    "depthwise_s1_b256": (63709.1 * 1.9995 + 113146.6 * 1.0000) * 1024,
    "maxpool_b64": (25477.1 * 1.9995 + 12544.0 * 1.0000) * 1024,
    "avgpool_b64": (2001.0 * 1.9995 + 80.0 * 1.0000) * 1024,
    "add_b64": (4723.0 * 1.9995 + 4704.0 * 1.0000) * 1024,
}


def traffic_still_valid(name):
    """Whether the kernel sources behind workload `name` are the ones its MEASURED_TRAFFIC entry was read on."""
    family = "thip_igemm.hip" if name.startswith(("fc_", "conv")) else "thip_bandwidth.hip"
    for source in ("thip_kernels_common.h", family):
        with open(os.path.join(ROOT, "torq-compiler_amd", "csrc", source), "rb") as f:
            if hashlib.sha256(f.read()).hexdigest() != TRAFFIC_SOURCES_SHA256[source]:
                return False
    return True


# The traffic shape of the benchmark's bandwidth rows for the streaming-floor calibration: 16-byte reads per 16-byte
# write (1, 2 or 4) and bytes written per launch.  The floor is what the fastest of a family of kernels with next to
# no arithmetic (1 to 8 items per thread, one pass or persistent, default or non-temporal cache policy) takes for the
# same bytes on the same buffers-larger-than-cache rotation.
STREAM_SHAPES = {
    "depthwise_b64": (4, 64 * 28 * 28 * 144), "depthwise_s1_b256": (1, 256 * 56 * 56 * 144), "maxpool_b64": (4, 64 * 56 * 56 * 64),
    "add_b64": (2, 64 * 56 * 56 * 24), "rescale_b64": (1, 64 * 56 * 56 * 24), "mul_b64": (2, 64 * 56 * 56 * 24),
}


def roofline(wl, bound, ms, name=None):
    traffic = MEASURED_TRAFFIC.get(name) if name in MEASURED_TRAFFIC and traffic_still_valid(name) else None
    traffic = None if traffic is None else int(round(traffic))
    if bound == "mfma":
        achieved = wl.ops / (ms * 1e-3) / 1e12
        return {"bound": "mfma", "achieved": round(achieved, 3), "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                "frac": round(achieved / PEAK_INT8_TOPS, 5), "traffic": traffic}
    achieved = wl.bytes / (ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": round(achieved, 2), "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": round(achieved / PEAK_HBM_GBS, 5), "traffic": traffic}


def verify_sample(loaded):
    """Checks the GPU result of the timed workload against the oracle (sampled rows for the big GEMMs)."""
    from oracle import oracle as orc
    from oracle.programs import assert_bf16_close, eval_network as oracle_network, eval_workload as oracle_eval
    wl = loaded.wl
    if wl.name.startswith("decoder_step"):
        import torq_compiler_amd as pkg
        return decoder_parity(pkg, loaded.dev, wl.attrs["batch"])
    got = loaded.output()
    if wl.name.startswith("mobilenet_v2"):
        n = min(4, wl.inputs[0].shape[0])
        import torq_compiler_amd as pkg
        return bool(np.array_equal(got[:n], oracle_network(pkg.workloads.mobilenet_v2_workload(batch=n))))
    if wl.name.startswith("fully_connected") and wl.inputs[0].shape[0] > 64:
        a = dict(wl.attrs)
        wts, sb = a.pop("weights"), a.pop("scale_bias")
        M = wl.inputs[0].shape[0]
        rows = np.unique(np.r_[0:16, M // 2:M // 2 + 16, M - 16:M])
        want = orc.fully_connected(wl.inputs[0][rows], wts, sb, **a)
        return bool(np.array_equal(got[rows], want))
    if wl.name.startswith("fcbf16") or wl.name.startswith("expandmm"):
        # tolerance row: one bf16 ULP, or the fp32 reordering error where the sum cancels
        f = lambda bits: np.abs(orc.from_bf16(bits).astype(np.float64))
        if wl.name.startswith("expandmm"):
            a = wl.attrs
            w16 = orc.expand_weights(a["weights"], a["scale"], a["qbias"], block_size=a["block"], output_min=a["expand_min"], output_max=a["expand_max"])
            mag = f(wl.inputs[0]) @ f(w16)
            got = got.reshape(mag.shape)
        else:
            mag = f(wl.inputs[0]) @ f(wl.attrs["weights"]).T + np.abs(wl.attrs["bias"])
        try:
            assert_bf16_close(got, oracle_eval(wl)[0].reshape(got.shape), wl.name, magnitude=mag)
        except AssertionError:
            return False
        return True
    return bool(np.array_equal(got, oracle_eval(wl)[0]))


def cpu_baseline(wl, target_seconds=10.0, single_thread_seconds=6.0):
    """Times the CPU oracle on a bounded sample of the default workload on this host's cores: with every core
    (`value`, `cores`) and with one thread (`single_thread`)."""
    from oracle import oracle as orc
    a = dict(wl.attrs)
    wts, sb = a.pop("weights"), a.pop("scale_bias")
    x = wl.inputs[0]
    M, K = x.shape
    N = wts.shape[0]

    def timed(seconds):
        rows = min(M, 4)
        t0 = time.perf_counter()
        orc.fully_connected(x[:rows], wts, sb, **a)
        dt = max(time.perf_counter() - t0, 1e-4)
        rows = int(min(M, max(rows, rows * 2.0 / dt)))  # about 2 s per pass
        passes, dt = 0, 0.0
        t0 = time.perf_counter()
        while dt < seconds:
            orc.fully_connected(x[:rows], wts, sb, **a)
            passes += 1
            dt = time.perf_counter() - t0
        return 2.0 * rows * passes * K * N / dt / 1e9, passes, rows, dt

    cores = orc.threads()
    gops, passes, rows, dt = timed(target_seconds)
    orc.set_threads(1)
    try:
        gops1, passes1, rows1, dt1 = timed(single_thread_seconds)
    finally:
        orc.set_threads(cores)
    what = "%d passes over the first %d of %d rows of the same (M,K,N)=(%d,%d,%d) fully_connected, %.1f s, C oracle"
    return {"value": round(gops, 2), "unit": "GOP/s", "cores": cores, "kind": "port",
            "sample": (what + " with OpenMP") % (passes, rows, M, M, K, N, dt),
            "single_thread": {"value": round(gops1, 2), "unit": "GOP/s", "cores": 1,
                              "sample": (what + ", one thread") % (passes1, rows1, M, M, K, N, dt1)}}


class PowerMeter:
    """Samples the card's power sensor (hwmon `power1_average` / `power1_input`, microwatts) from a thread.  A machine that
    does not show the sensor gives None everywhere.  With several cards present the busiest one is reported."""

    def __init__(self, period=0.005):
        import glob
        self.paths = sorted(p for name in ("power1_average", "power1_input")
                            for p in glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/" + name))
        self.period = period
        self.samples = []   # (time.time(), [watts per sensor])
        self.thread = None

    def cap_watts(self):
        caps = []
        for p in self.paths:
            try:
                caps.append(int(open(os.path.join(os.path.dirname(p), "power1_cap")).read()) / 1e6)
            except (OSError, ValueError):
                pass
        return max(caps) if caps else None

    def _loop(self):
        while self.running:
            row = []
            for p in self.paths:
                try:
                    row.append(int(open(p).read()) / 1e6)
                except (OSError, ValueError):
                    row.append(0.0)
            self.samples.append((time.time(), row))
            time.sleep(self.period)

    def __enter__(self):
        import threading
        self.samples, self.running = [], bool(self.paths)
        if self.running:
            self.thread = threading.Thread(target=self._loop, daemon=True)
            self.thread.start()
        return self

    def __exit__(self, *exc):
        self.running = False
        if self.thread:
            self.thread.join()

    def mean_watts(self, t0, t1):
        """Mean over the second half of [t0, t1] (the sensor itself averages over a while)."""
        rows = [r for t, r in self.samples if t0 + 0.5 * (t1 - t0) <= t <= t1]
        if not rows:
            return None
        return round(max(float(np.mean([r[i] for r in rows])) for i in range(len(self.paths))), 1)


def mfma_calibration(pkg, dev, wl, args):
    """What bounds the headline GEMM on this card, measured in this run (TOP/s, 1 multiply-add = 2 ops), and what
    the card draws meanwhile: every leg is repeated for `leg_seconds` under the power sensor."""
    out = {"unit": "TOP/s", "published_peak": PEAK_INT8_TOPS}
    meter = PowerMeter()
    leg_seconds = max(0.0, args.leg_seconds)
    power = {"unit": "W", "sensor": meter.paths[0] if meter.paths else None, "cap": meter.cap_watts(), "leg_seconds": leg_seconds}

    def leg(label, fn):
        """Median of fn() over the leg; the power goes into power[label]."""
        results = []
        with meter:
            t0 = time.time()
            results.append(fn())
            while time.time() - t0 < leg_seconds:
                results.append(fn())
            t1 = time.time()
        power[label] = meter.mean_watts(t0, t1)
        return float(np.median(results))

    leg("idle", lambda: time.sleep(0.05) or 0.0)
    # the matrix cores with nothing else going on: every CU busy (256 workgroups of 4 waves), and 32 workgroups only
    # (an eighth of the chip: far below the power limit, so this is the clock-limited rate of one CU)
    out["mfma_only_constant_operands"] = round(leg("mfma_only_constant_operands", lambda: dev.mfma_rate(False, 256, 12000)), 1)
    out["mfma_only_random_operands"] = round(leg("mfma_only_random_operands", lambda: dev.mfma_rate(True, 256, 12000)), 1)
    out["mfma_only_random_operands_32_of_256_cus_scaled"] = round(
        leg("mfma_only_random_operands_32_of_256_cus", lambda: dev.mfma_rate(True, 32, 12000)) * 8, 1)
    # the same GEMM kernel on all-zero operands (nothing toggles) against the benchmark's uniform random bytes
    M, K = wl.inputs[0].shape
    N = wl.attrs["weights"].shape[0]
    for label, zeros in (("gemm_random_data", False), ("gemm_zero_data", True)):
        o = Loaded(pkg, dev, pkg.workloads.fully_connected_workload(M, K, N, zeros=zeros))
        o.run(args.warmup)
        ms = leg(label, lambda: o.run(args.steps))
        out[label] = {"us": round(ms * 1e3, 2), "TOP/s": round(o.wl.ops / (ms * 1e-3) / 1e12, 1), "kernel": o.exe.op_kernels()[0]}
        o.close()
    out["gemm_over_mfma_only_random"] = round(out["gemm_random_data"]["TOP/s"] / out["mfma_only_random_operands"], 3)
    if args.library_gemm:
        # in a process of its own: PyTorch brings its own HIP runtime, which does not share a process with this library's
        import subprocess
        script = ("import torch, json, time\n"
                  "M, K, N, W, S, T = %d, %d, %d, %d, %d, %f\n"
                  "a = torch.randint(-128, 128, (M, K), dtype=torch.int8, device='cuda:0')\n"
                  "bt = torch.randint(-128, 128, (N, K), dtype=torch.int8, device='cuda:0').t()\n"
                  "for _ in range(W): torch._int_mm(a, bt)\n"
                  "torch.cuda.synchronize()\n"
                  "e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)\n"
                  "t0, ms = time.time(), []\n"
                  "while not ms or time.time() - t0 < T:\n"
                  "    e0.record()\n"
                  "    for _ in range(S): torch._int_mm(a, bt)\n"
                  "    e1.record(); torch.cuda.synchronize()\n"
                  "    ms.append(e0.elapsed_time(e1) / S)\n"
                  "ms.sort()\n"
                  "print(json.dumps({'ms': ms[len(ms) // 2], 't0': t0, 't1': time.time()}))\n") % (M, K, N, max(args.warmup, 5), args.steps, leg_seconds)
        try:
            with meter:
                done = subprocess.run([sys.executable, "-c", script], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
            res = json.loads(done.stdout.strip().splitlines()[-1])
            ms = res["ms"]
            power["library_int_mm_random_data"] = meter.mean_watts(res["t0"], res["t1"])
            out["library_int_mm_random_data"] = {"us": round(ms * 1e3, 2), "TOP/s": round(2.0 * M * K * N / (ms * 1e-3) / 1e12, 1),
                                                 "what": "torch._int_mm (hipBLASLt) in a child process: int32 result, no requant, [N,K] weights like ours"}
        except Exception as ex:  # the comparison is optional
            out["library_int_mm_random_data"] = "unavailable: %r" % (ex,)
    out["power"] = power
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="fc_4096x4096x4096")
    ap.add_argument("--precondition-ms", type=float, default=200.0,
                    help="untimed dispatches of the workload for this long before its warm-up steps, so that the card has left its idle "
                         "clocks when the timed steps start (0 switches it off); reported as config.clock_preconditioning_ms")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-others", action="store_true", help="skip the brief per-op measurements")
    ap.add_argument("--mfma-calibration", action="store_true",
                    help="also measure what bounds the int8 GEMM on this card: the matrix cores alone on constant and on random operands, "
                         "the same GEMM on all-zero data, and (with --library-gemm) the vendor library's int8 GEMM")
    ap.add_argument("--leg-seconds", type=float, default=1.5,
                    help="with --mfma-calibration: every measurement is repeated for this long (the clocks settle, the power sensor "
                         "averages); 0 = once each, for a short run under a profiler")
    ap.add_argument("--library-gemm", action="store_true", help="with --mfma-calibration: time torch._int_mm (hipBLASLt) on the same shape")
    ap.add_argument("--cold", action="store_true",
                    help="time --workload on rotating copies of its buffers (together larger than the last-level cache), as the "
                         "bandwidth rows of per_op are timed")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy (a 1x1 max pool), to scale rocprofv3's FETCH_SIZE / WRITE_SIZE by")
    ap.add_argument("--stream-floor", action="store_true",
                    help="only the streaming-floor calibration: the fastest member of the family for the traffic shape of every "
                         "bandwidth row and for a 256 MiB copy, cold; one JSON line (for a run under rocprofv3)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    pkg = import_package()
    if args.stream_floor:
        dev = pkg.Device(0)
        rows = {}
        for name, (rd, wbytes) in list(STREAM_SHAPES.items()) + [("copy_256MiB", (1, 256 << 20))]:
            wbytes = wbytes // 16 * 16
            us, kernel = min(dev.stream_floor(rd, wbytes, cold=True, variant=True) for _ in range(3))
            moved = (rd + 1) * wbytes
            rows[name] = {"reads_per_write": rd, "bytes": moved, "us": round(us, 2), "kernel": kernel, "GB/s": round(moved / us / 1e3, 1),
                          "frac": round(moved / us / 1e3 / PEAK_HBM_GBS, 3)}
        dev.close()
        print(json.dumps({"streaming_floor": rows}))
        return
    table = workload_table(pkg)
    nets = network_table(pkg)
    if args.workload in nets:
        table = dict(table)
        table[args.workload] = nets[args.workload]
    if args.workload not in table:
        sys.exit("unknown workload %s; choose from %s" % (args.workload, ", ".join(table)))
    dev = pkg.Device(0)

    make, bound = table[args.workload]
    wl = make()
    loaded = Loaded(pkg, dev, wl)
    kernels = loaded.exe.op_kernels()
    pre_ms = max(0.0, args.precondition_ms)
    loaded.precondition(pre_ms)
    if args.warmup > 0:
        loaded.run(args.warmup)
    dev.synchronize()
    t0 = time.perf_counter()
    main_sets = 1
    if args.cold:
        ev_ms, main_sets = loaded.run_cold(args.steps, pre_ms)
    else:
        ev_ms = loaded.run(args.steps)      # HIP events on the executable's stream around the K dispatches
    dev.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    if args.cold:
        wall_ms = ev_ms  # the wall clock above also holds the upload of the extra buffer sets
    # the CPU leg (--no-cpu skips all of it): the oracle as the timed baseline and as the checker of this run's results
    ok = None if args.no_cpu else verify_sample(loaded)
    loaded.close()
    if args.copy_calibration:
        # a 1x1 stride-1 max pool over the whole int8 range is a plain copy: 256 MiB read, 256 MiB written
        prog = pkg.Program()
        shape = (1, 4096, 4096, 16)
        src = prog.binding(0, shape)
        prog.maxpool2d(src, input_zp=-128, output_min=-128, output_max=127, stride=(1, 1), pad=(0, 0, 0, 0), kernel=(1, 1),
                       init=prog.binding(1, shape), nhwc_input=True)
        exe = pkg.Executable(dev, prog.serialize())
        host = np.zeros(shape, dtype=np.int8)
        ptrs = [dev.upload(host), dev.upload(host)]
        exe.time_device(ptrs, [host.nbytes, host.nbytes], 3)
        exe.close()
        for ptr in ptrs:
            dev.free(ptr)

    calibration = None
    if args.mfma_calibration:
        calibration = mfma_calibration(pkg, dev, wl, args)

    per_op = {}
    if not args.no_others:
        for name, (mk, bnd) in table.items():
            if name == args.workload:
                continue
            o = Loaded(pkg, dev, mk())
            o.precondition(pre_ms)
            o.run(5)
            warm = min(o.run(50) for _ in range(3))  # best of three: 50 dispatches of a 3 us kernel are over before a hiccup of the host's is
            names = o.exe.op_kernels()
            row = {"kernel": names[-1 if "transpose" in names[0] else 0], "bound": bnd}
            if bnd == "hbm":
                # what the roofline fraction is quoted on: operands cold in every dispatch; the repeated dispatch of one
                # buffer set (served by the last-level cache where it fits) is reported next to it
                ms, sets = o.run_cold(50, pre_ms, repeats=3)
                row.update({"us": round(ms * 1e3, 2), "us_cache_warm": round(warm * 1e3, 2), "buffer_sets": sets})
                if name in STREAM_SHAPES:
                    rd, wbytes = STREAM_SHAPES[name]
                    wbytes = wbytes // 16 * 16
                    floor_us, floor_kernel = min(dev.stream_floor(rd, wbytes, cold=True, variant=True) for _ in range(3))  # the first call meets a card that has idled
                    row["streaming_floor_us"] = round(floor_us, 2)
                    row["streaming_floor_kernel"] = floor_kernel
                    row["frac_of_streaming_floor"] = round(floor_us / (ms * 1e3), 3)
            else:
                ms = warm
                row["us"] = round(ms * 1e3, 2)
            r = roofline(o.wl, bnd, ms, name)
            row.update({"GOP/s": round(o.wl.ops / (ms * 1e-3) / 1e9, 1), "GB/s": round(o.wl.bytes / (ms * 1e-3) / 1e9, 1), "frac": r["frac"]})
            if r["traffic"] is not None:
                row["traffic"] = r["traffic"]  # HBM bytes per launch from the rocprofv3 counters (MEASURED_TRAFFIC)
            if not args.no_cpu:
                row["parity_checked"] = verify_sample(o)
                ok = ok and row["parity_checked"]
            per_op[name] = row
            o.close()

    mbv2 = {}
    if not args.no_others:
        if not args.no_cpu:
            from oracle.programs import eval_network as oracle_network
        for batch in (1, 32, 256):
            o = Loaded(pkg, dev, pkg.workloads.mobilenet_v2_workload(batch=batch))
            o.precondition(pre_ms)
            o.run(2)
            ms = min(o.run(10 if batch > 1 else 30) for _ in range(3))
            same = None
            if not args.no_cpu:
                check = pkg.workloads.mobilenet_v2_workload(batch=min(batch, 4))  # same seed: same weights, first images
                same = bool(np.array_equal(o.output()[:min(batch, 4)], oracle_network(check)))
            mbv2["batch_%d" % batch] = {"ms": round(ms, 4), "images_per_s": round(batch / (ms * 1e-3), 1),
                                       "GOP/s": round(o.wl.ops / (ms * 1e-3) / 1e9, 1), "kernels": len(o.exe.op_kernels()),
                                       "parity_checked": same}
            ok = ok and same if same is not None else ok
            o.close()

    decoder = {}
    if not args.no_others:
        for batch in DECODER_BATCHES:
            decoder["batch_%d" % batch] = decoder_row(pkg, dev, batch, pre_ms, not args.no_cpu)
            if not args.no_cpu:
                ok = ok and decoder["batch_%d" % batch]["parity_checked"]

    result = {
        "metric": "int8 GOP/s (fully_connected with fused requant), 1 MAC = 2 ops",
        "value": round(wl.ops / (wall_ms * 1e-3) / 1e9, 1),
        "unit": "GOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.workload.startswith(("fcbf16", "expandmm", "decoder")) else "int8",
        "data": "synthetic",
        "config": {"workload": args.workload, "kernels": kernels, "parity_checked": ok,
                   "algorithmic_ops": wl.ops, "algorithmic_bytes": wl.bytes, "buffer_sets": main_sets,
                   "clock_preconditioning_ms": pre_ms},
        "roofline": dict(roofline(wl, bound, ev_ms, args.workload), kernel=kernels[0], kernel_ms=round(ev_ms, 5)),
    }
    if not args.no_cpu and args.workload.startswith("fc_"):
        result["cpu_baseline"] = cpu_baseline(wl)
    if calibration:
        result["mfma_calibration"] = calibration
    if per_op:
        result["per_op"] = per_op
    if mbv2:
        result["mobilenet_v2_int8_224"] = mbv2
    if decoder:
        result["decoder_step"] = decoder
    dev.close()
    print(json.dumps(result))
    if ok is False:
        sys.exit("GPU result differs from the oracle")


if __name__ == "__main__":
    main()
