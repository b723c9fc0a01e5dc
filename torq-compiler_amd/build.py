"""Builds ``libthip.so`` (HIP kernels + driver + emitter behind the C-ABI) for gfx950.

hipcc cross-compiles without a GPU.  The library is written next to this file so
that it travels with the source tree; nothing is installed.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libthip.so")
OBJ_DIR = os.path.join(HERE, "build")

SOURCES = ["thip_kernels.hip", "thip_driver.cpp", "thip_emitter.cpp", "thip_validate.cpp", "thip_status.cpp"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = ["-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
          "--offload-arch=gfx950",
          # packed FP32 instruction selection stays off for every device pass
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          # no v_dot4c_i32_i8: its accumulator is tied to the destination, so every dot-product chain that starts from
          # a value it must keep (the bias) costs a v_mov per output; v_dot4_i32_i8 takes the addend as a third operand
          "-Xclang", "-target-feature", "-Xclang", "-dot6-insts"]


def _compile(src, extra):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC] + COMMON + extra + ["-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l and "dot6-insts" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
    return obj, out


def build(verbose=False, extra=()):
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=4) as pool:
        results = list(pool.map(lambda s: _compile(s, list(extra)), SOURCES))
    objs = [r[0] for r in results]
    if verbose:
        for _, out in results:
            if out.strip():
                print(out)
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n" + proc.stdout)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True, extra=sys.argv[1:]))
