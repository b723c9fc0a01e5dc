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

SOURCES = ["thip_igemm.hip", "thip_bandwidth.hip", "thip_bf16.hip", "thip_decode.hip", "thip_device_util.hip", "thip_driver.cpp", "thip_emitter.cpp",
           "thip_validate.cpp", "thip_status.cpp"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = ["-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
          "--offload-arch=gfx950",
          # packed FP32 instruction selection stays off for every device pass
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          # no v_dot4c_i32_i8: its accumulator is tied to the destination, so every dot-product chain that starts from
          # a value it must keep (the bias) costs a v_mov per output; v_dot4_i32_i8 takes the addend as a third operand
          "-Xclang", "-target-feature", "-Xclang", "-dot6-insts"]


HEADERS = ["thip_kernels.h", "thip_kernels_common.h", "thip_descriptor.h", "thip_status.h", "thip_validate.h"]


def _up_to_date(src, obj):
    if not os.path.exists(obj):
        return False
    deps = [os.path.join(CSRC, src)] + [os.path.join(CSRC, h) for h in HEADERS] + [os.path.join(os.path.dirname(HERE), "include", "thip.h"), __file__]
    return all(os.path.getmtime(d) <= os.path.getmtime(obj) for d in deps if os.path.exists(d))


def _compile(src, extra, force=True):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    if not force and _up_to_date(src, obj):
        return obj, ""
    cmd = [HIPCC] + COMMON + extra + ["-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l and "dot6-insts" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
    return obj, out


def build(verbose=False, extra=(), force=True):
    """Compiles every source and links the library.  force=False (the command line's default: a developer's edit
    loop) recompiles only sources older than their object file."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=8) as pool:
        results = list(pool.map(lambda s: _compile(s, list(extra), force), SOURCES))
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
    args = sys.argv[1:]
    print(build(verbose=True, extra=[a for a in args if a != "--force"], force="--force" in args))
