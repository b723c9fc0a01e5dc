"""MI355X (gfx950) backend for the quantized TorqHL operator path.

``runtime``  ctypes binding of the C-ABI (include/thip.h) -- device, executable, dispatch.
``torq_hl``  host-side mirror of the TorqHL ops; builds a program and serialises it.
``workloads`` seeded synthetic workloads at the benchmark shapes.

The compute lives in ``libthip.so`` (HIP kernels + C++ driver + C++ emitter, built by
``build.py``).  There is no CPU execution path in this package.
"""
from . import runtime, torq_hl, workloads  # noqa: F401
from .runtime import Device, Executable, ThipError  # noqa: F401
from .torq_hl import Program  # noqa: F401
