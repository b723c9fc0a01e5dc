"""Corrupt descriptors and hostile op attributes must come back as a status, never as a crash.

Two layers, both on the CPU: (1) mutated blobs of real workloads through the shipped library's
thip_descriptor_validate / thip_infer_format; (2) tests/fuzz/fuzz_host.cpp, a stand-alone driver over the emitter, the
validation and the oracle, compiled with -fsanitize=address,undefined (the host sources only: none of them calls HIP)
and run as a subprocess: any sanitizer report or non-zero exit fails the test.
"""
import ctypes
import os
import shutil
import subprocess

import numpy as np
import pytest

import desc_interp
from torq_compiler_amd import runtime, workloads as w

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "torq-compiler_amd", "csrc")


def _validate(blob_bytes, size=None):
    buf = ctypes.create_string_buffer(bytes(blob_bytes), len(blob_bytes))  # 8-byte aligned or better
    assert ctypes.addressof(buf) % 8 == 0
    code = runtime.lib().thip_descriptor_validate(buf, len(blob_bytes) if size is None else size)
    fmt = ctypes.create_string_buffer(32)
    inferred = ctypes.c_size_t()
    code2 = runtime.lib().thip_infer_format(buf, len(blob_bytes) if size is None else size, 32, fmt, ctypes.byref(inferred))
    assert (code == runtime.OK) == (code2 == runtime.OK)
    return code


@pytest.mark.parametrize("make", [
    lambda: w.conv2d_workload(N=1, H=9, W=9, C=3, O=8, realistic=True), lambda: w.conv2d_workload(N=1, H=8, W=8, C=24, O=16, realistic=True),
    lambda: w.depthwise_workload(N=1, H=12, W=12, C=32), lambda: w.fully_connected_workload(40, 72, 20, realistic=True),
    lambda: w.matmul_workload(2, 9, 61, 37), lambda: w.fully_connected_bf16_workload(1, 6912, 256),
    lambda: w.expand_weights_workload(M=4, K=256, N=96, block=32), lambda: w.pointwise_add_workload(N=1, H=16, W=16, C=32, O=32),
    lambda: w.mobilenet_v2_workload(batch=1, resolution=32, classes=10, width=0.25),
    lambda: w.grouped_linear_workload(mode="pair", zero_points=True), lambda: w.grouped_linear_workload(mode="concat", M=32),
    lambda: w.grouped_linear_workload(mode="residual", K=256, N=256), lambda: w.attention_workload(B=2, H=4, D=64, T=128, D2=64),
    lambda: w.decoder_step_workload(batch=3, layers=1, hidden=256, heads=2, head_dim=64, ffn=384, vocab=512, cache_len=64),
], ids=["conv_runs", "conv_gather", "depthwise", "fc", "matmul", "fc_bf16_splitk", "expand_mm", "conv_add", "network", "linear_pair", "linear_concat",
        "linear_residual", "attention", "decoder_step"])
def test_mutated_descriptors_return_a_status(make):
    blob = bytearray(make().program.serialize())
    assert _validate(blob) == runtime.OK
    header = np.frombuffer(bytes(blob[:88]), dtype="<u8")
    structured = int(header[8])  # data_offset: header, records and tables lie below it
    # the grouped linear records keep their per-matrix operand references in a constant (their `table`): mutate those too
    d = desc_interp.Descriptor(bytes(blob))
    ext = [(structured + int(d.consts[int(o["table"]["index"])]["offset"]) + int(o["table"]["offset"]), 224) for o in d.ops if int(o["kind"]) == 15]
    rng = np.random.default_rng(len(blob))
    outcomes = set()
    for _ in range(400):
        bad = bytearray(blob)
        how = int(rng.integers(0, 5 if ext else 4))
        size = None
        if how == 0:
            size = int(rng.integers(0, len(bad)))
        elif how == 1:
            for _ in range(int(rng.integers(1, 4))):
                bad[int(rng.integers(0, 88))] ^= 1 << int(rng.integers(0, 8))
        elif how == 2:
            for _ in range(int(rng.integers(1, 4))):
                bad[int(rng.integers(0, structured))] ^= 1 << int(rng.integers(0, 8))
        elif how == 3:
            at = int(rng.integers(0, structured // 4)) * 4
            bad[at:at + 4] = int(rng.choice([0, 0xffffffff, 0x7fffffff, 0x80000000, int(rng.integers(0, 1 << 32))])).to_bytes(4, "little")
        else:
            start, size_ext = ext[int(rng.integers(0, len(ext)))]
            at = start + int(rng.integers(0, size_ext // 4)) * 4
            bad[at:at + 4] = int(rng.choice([0, 0xffffffff, 0x7fffffff, 0x80000000, 3, int(rng.integers(0, 1 << 32))])).to_bytes(4, "little")
        outcomes.add(_validate(bad, size))
    assert runtime.INVALID_ARGUMENT in outcomes  # and whatever else came back was a status: the process is still here


def test_emitter_validation_and_oracle_under_sanitizers(tmp_path):
    gxx = shutil.which("g++")
    assert gxx, "g++ is needed for the sanitizer build of the host sources"
    exe = str(tmp_path / "fuzz_host")
    cmd = [gxx, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-static-libasan", "-fno-sanitize-recover=undefined", "-fopenmp", "-w",
           "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", "-I" + CSRC,
           os.path.join(ROOT, "tests", "fuzz", "fuzz_host.cpp"), os.path.join(CSRC, "thip_emitter.cpp"), os.path.join(CSRC, "thip_validate.cpp"),
           os.path.join(CSRC, "thip_status.cpp"), "-x", "c", os.path.join(ROOT, "oracle", "torq_oracle.c"), "-o", exe]
    built = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert built.returncode == 0, built.stdout[-3000:]
    # the sanitizer runtime is linked statically, so it does not care where it stands among the process's libraries
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:verify_asan_link_order=0", UBSAN_OPTIONS="print_stacktrace=1", OMP_NUM_THREADS="2")
    run = subprocess.run([exe, "240", "50"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env, timeout=600)
    assert run.returncode == 0 and "fuzz ok" in run.stdout and "runtime error" not in run.stdout and "AddressSanitizer" not in run.stdout, run.stdout[-4000:]
